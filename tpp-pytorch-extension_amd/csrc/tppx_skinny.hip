// Decode-shape kernels (up to 64 rows) with the K reduction kept inside the workgroup.
//
// One workgroup owns a few consecutive 16-channel weight tiles and all of K
// (or one of a few K parts, see finish_split); its 8 or 16 waves split K
// into contiguous ranges.  A wave streams the native 1 KiB tiles of its range
// straight from HBM into registers (one 128-bit load per lane and tile, a ring
// of PF k-tiles in flight, issued before anything that could wait), feeds the
// 16x16 MFMA, and at the end the waves' partial tiles are summed through LDS
// in a fixed order (deterministic) and the fused epilogue runs.  No atomics
// on data.  The kernels differ in how the activation operand gets there:
//   skinny_qint8_kernel     int8 activations already in MFMA operand order in
//                           global memory (written by the quantiser), 17..64 rows
//   skinny_qint8_fq_kernel  bf16 activations quantised by the consuming wave into
//                           wave-private LDS, up to 16 rows
//   skinny_mxfp4_xl_kernel  the wave's whole K slice staged once in LDS, up to
//                           16 rows; optional RMSNorm in front
//   skinny_mxfp4_x4_kernel  the same with only 4 rows kept, for long K
//   skinny_mxfp4_mg_kernel  activations streamed through LDS one K tile at a
//                           time, 1, 2 or 4 row groups of 16
//
// MFMA operand convention (A = activations, B = weights):
//   lane l supplies row/col (l & 15) and K group (l >> 4);
//   result register r of lane l is D[m = (l >> 4) * 4 + r][n = l & 15].
#include <mutex>

#include "tppx_common.h"
#include "tppx_launch.h"

namespace tppx {

__device__ __forceinline__ bf16x8 sk_cvt_fp4x8(uint32_t codes, float scale) {
  bf16x2 c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 0);
  bf16x2 c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 1);
  bf16x2 c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 2);
  bf16x2 c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 3);
  bf16x8 w;
  w[0] = c0[0]; w[1] = c0[1]; w[2] = c1[0]; w[3] = c1[1];
  w[4] = c2[0]; w[5] = c2[1]; w[6] = c3[0]; w[7] = c3[1];
  return w;
}

// two floats -> two bf16 (round to nearest even) in one dword: the hardware conversion, one instruction per pair
// (the normalisation in front of a GEMM converts M x K values in EVERY workgroup)
__device__ __forceinline__ uint32_t sk_pack_bf16(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  const bf16x2 v = __builtin_convertvector(f32x2{lo, hi}, bf16x2);
  return __builtin_bit_cast(uint32_t, v);
}

// floor(a * b / c) for the K-range splits: a * b stays far below 2^31 (at most 2^18 tiles times 16 waves or 4 parts),
// so one 32-bit unsigned division does (the 64-bit form is a hundred instructions and four branches per use, and stood
// in front of every kernel's first weight request).
__device__ __forceinline__ int sk_share(int a, int b, int c) {
  return (int)(((unsigned int)a * (unsigned int)b) / (unsigned int)c);
}

// the same for the K slices across workgroups: their number is 1, 2 or 4 (the launchers check), so a shift does
__device__ __forceinline__ int sk_share_pow2(int a, int b, int c) {
  return (int)(((unsigned int)a * (unsigned int)b) >> __builtin_ctz((unsigned int)c));
}

__device__ __forceinline__ int sk_find_seg(const DecodeParams& p, int grp) {
  int s = 0;
#pragma unroll
  for (int i = 1; i < TPPX_MAX_SEGS; i++)
    if (i < p.n_seg && grp >= p.seg[i].grp0)
      s = i;
  return s;
}

// Arrival counters of the launches that split K across workgroups: one per (block row, channel group), all zero
// between launches (the counting instruction wraps to zero on the last arrival).  A launch takes a window of
// them that the host hands out in rotation, so launches in flight at the same time do not share counters as long
// as fewer than SK_TICKETS counters are in use at once.
constexpr int SK_TICKETS = 16384;
__device__ unsigned int sk_split_tickets[SK_TICKETS];

// LDS reduction over the waves of the workgroup + fused epilogue.
// red layout: [wave][(a*MG + mg)*256 + r*64 + lane]; every thread finishes
// EPT = NACC_OUT*MG*256 / blockDim outputs whose post-op inputs it fetched
// before the main loop.
// FIXW: the number of waves of the workgroup where the kernel knows it at compile time (0: read from the launch).  The
// cross-wave sums then unroll completely and all of a thread's LDS reads are issued before the first wait; with a
// run-time count the compiler waited for the LDS once per output and batch of eight (36 waits of an LDS round trip
// each in the 64-row gate/up epilogue: 1.3 us per half).
template <int MG, int NACC, bool DUAL, int MINW, int FIXW = 0>
struct SkEpilogue {
  static __device__ __forceinline__ int nthreads() { return FIXW ? FIXW * 64 : (int)blockDim.x; }
  static __device__ __forceinline__ int nwaves() { return FIXW ? FIXW : (int)(blockDim.x >> 6); }
  static constexpr int ELEMS = NACC * MG * 256;
  static constexpr int OUT = DUAL ? ELEMS / 2 : ELEMS;
  // outputs per thread; the launcher never uses fewer than MINW waves
  static constexpr int MAXE = (OUT + MINW * 64 - 1) / (MINW * 64);
  int off[MAXE]; // element offset of the output (the launcher checks M * N < 2^31), or -1: nothing to store
  uint32_t in1[MAXE], in2[MAXE];
  uint32_t bias[MAXE], bias2[MAXE]; // bf16 bits, converted at use: a conversion here would wait for the load at once

  bool has_bias, has_bias2, has_in1, has_in2; // uniform: which of the arrays below hold real inputs

  // Requests the post-op inputs of this thread's outputs.  No branch around any load: an absent input is read from the
  // output tensor instead (valid memory of the same extent; the value is dropped in settle()).  A load inside a
  // conditional makes the compiler wait for every outstanding load at the join, which here stood between the
  // activations and the first weight request of the kernel.
  __device__ __forceinline__ void prefetch_flat(const DecodeParams& p, const DecodeSeg& sg, int ltile0, int m0) {
    // Everything the loop needs of the descriptors is read ONCE into scalars here: left to the use sites, every
    // element's offset arithmetic fetched its fields again behind branches of its own (in the 64-row kernels 43 scalar
    // loads, 29 waits and 45 branches stood in front of the first weight request).  The QINT8 kernels never split
    // their output over several matrices (DecodeSeg::split1 is the MXFP4 q/k/v launch's), so the offset is m * N + n.
    const int M = p.M, N = sg.N, tiles = sg.tiles;
    has_bias = sg.bias != nullptr;
    has_bias2 = DUAL && p.seg[1].bias != nullptr;
    has_in1 = sg.post_in != nullptr;
    has_in2 = sg.post_in2 != nullptr;
    const uint16_t* pb = has_bias ? sg.bias : sg.y;
    const uint16_t* pb2 = has_bias2 ? p.seg[1].bias : sg.y;
    const uint16_t* pi1 = has_in1 ? sg.post_in : sg.y;
    const uint16_t* pi2 = has_in2 ? sg.post_in2 : sg.y;
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      const int e = threadIdx.x + i * nthreads();
      const int l = e & 63, r = (e >> 6) & 3, mg = (e >> 8) % MG, a = (e >> 8) / MG;
      const int m = m0 + mg * 16 + (l >> 4) * 4 + r;
      const int n = (ltile0 + a) * 16 + (l & 15);
      const bool valid = e < OUT && m < M && (ltile0 + a) < tiles;
      const int o = valid ? m * N + n : 0, nn = valid ? n : 0;
      off[i] = valid ? o : -1;
      bias[i] = pb[nn];
      bias2[i] = DUAL ? pb2[nn] : 0;
      in1[i] = DUAL ? 0 : pi1[o];
      in2[i] = DUAL ? 0 : pi2[o];
    }
  }

  // The same with each input's loads under a (uniform) condition: fewer requests, for the kernels that place their
  // own waits by count (the MXFP4 ones) or issue this late.  Measured on the 7B decode step: the unconditional form
  // costs those kernels 0.3 us each.
  __device__ __forceinline__ void prefetch(const DecodeParams& p, const DecodeSeg& sg, int ltile0, int m0) {
    has_bias = has_bias2 = has_in1 = has_in2 = true; // absent inputs are zeros already
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      const int e = threadIdx.x + i * nthreads();
      in1[i] = in2[i] = 0;
      bias[i] = bias2[i] = 0;
      off[i] = -1;
      if (e < OUT) {
        const int l = e & 63, r = (e >> 6) & 3, mg = (e >> 8) % MG, a = (e >> 8) / MG;
        const int m = m0 + mg * 16 + (l >> 4) * 4 + r;
        const int n = (ltile0 + a) * 16 + (l & 15);
        if (m < p.M && (ltile0 + a) < sg.tiles) {
          off[i] = seg_out_offset(sg, p.M, m, n);
          if (sg.bias)
            bias[i] = sg.bias[n];
          if (DUAL && p.seg[1].bias)
            bias2[i] = p.seg[1].bias[n];
          if (sg.post_in)
            in1[i] = sg.post_in[off[i]];
          if (sg.post_in2)
            in2[i] = sg.post_in2[off[i]];
        }
      }
    }
  }

  // first thing after the main loop: drop what was read in place of an absent input
  __device__ __forceinline__ void settle() {
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      bias[i] = has_bias ? bias[i] : 0;
      bias2[i] = has_bias2 ? bias2[i] : 0;
      in1[i] = has_in1 ? in1[i] : 0;
      in2[i] = has_in2 ? in2[i] : 0;
    }
  }

  // The same with half the scratch for the gate/up pair: the gate tiles are reduced first, then the up tiles
  // (same sums in the same order as finish()).  stride >= ELEMS / 2.
  __device__ __forceinline__ void finish_halves(const DecodeSeg& sg, f32x4 (&acc)[NACC][MG], float* red, int stride = ELEMS / 2) {
    static_assert(DUAL, "two reduction rounds are for the gate/up pair");
    settle();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int W = nwaves();
    float* mine = red + wave * stride;
    float v[2][MAXE];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      if (h)
        __syncthreads(); // everybody has read the gate sums
#pragma unroll
      for (int a = 0; a < NACC / 2; a++)
#pragma unroll
        for (int mg = 0; mg < MG; mg++)
#pragma unroll
          for (int r = 0; r < 4; r++)
            mine[(a * MG + mg) * 256 + r * 64 + lane] = acc[h * (NACC / 2) + a][mg][r];
      __syncthreads();
      // (no branch per output here or below: slots past the outputs repeat the last one and are not stored, so the
      // outputs' LDS reads and their SiLU / multiply chains interleave instead of running one after the other)
#pragma unroll
      for (int i = 0; i < MAXE; i++) {
        const int e = min((int)threadIdx.x + i * nthreads(), OUT - 1);
        v[h][i] = 0.f;
#pragma unroll
        for (int w = 0; w < (FIXW ? FIXW : W); w++)
          v[h][i] += red[w * stride + e];
      }
    }
    uint32_t out[MAXE];
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      const uint32_t gact = apply_post_bits(v[0][i] + bf16_bits_to_f32(bias[i]), TPPX_POST_SILU, 0, 0, 1.0f);
      out[i] = apply_post_bits(v[1][i] + bf16_bits_to_f32(bias2[i]), TPPX_POST_MUL, gact, 0, 1.0f);
    }
#pragma unroll
    for (int i = 0; i < MAXE; i++)
      if (off[i] >= 0)
        sg.y[off[i]] = (uint16_t)out[i];
  }

  // Row sums of squares of this workgroup's outputs (MG == 1): ov[i] = the rounded output of slot i as a float, 0
  // where nothing was stored.  Called by every thread of the workgroup; entry [row][blockIdx.x] of the [16][256]
  // table gets the sum over this workgroup's channel tiles in a fixed order, and workgroup 0 zeroes the slots past
  // the grid.
  __device__ __forceinline__ void leave_row_sums(const float (&ov)[MAXE], float* sumsq, int M) {
    __shared__ float sq_s[16 * NACC];
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      const int e = threadIdx.x + i * nthreads();
      if (e < OUT) { // wave-uniform: e < OUT holds for whole waves
        float sq = ov[i] * ov[i];
        // the 16 lanes of a DPP row hold the 16 channels of one (row, tile) pair
        sq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sq), 0xB1, 0xf, 0xf, true));
        sq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sq), 0x4E, 0xf, 0xf, true));
        sq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sq), 0x141, 0xf, 0xf, true));
        sq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sq), 0x140, 0xf, 0xf, true));
        if ((e & 15) == 0)
          sq_s[(((e & 63) >> 4) * 4 + ((e >> 6) & 3)) * NACC + (e >> 8)] = sq; // [row][tile]
      }
    }
    __syncthreads();
    if (threadIdx.x < 16 && (int)threadIdx.x < M) {
      float tot = 0.f;
#pragma unroll
      for (int a = 0; a < NACC; a++)
        tot += sq_s[threadIdx.x * NACC + a];
      sumsq[threadIdx.x * 256 + blockIdx.x] = tot;
    }
    if (blockIdx.x == 0)
      for (int j = (int)gridDim.x + (int)threadIdx.x; j < 256 * min(M, 16); j += (int)blockDim.x) {
        const int row = j >> 8, part = j & 255; // slots gridDim.x .. 255 of every row (j walks a superset)
        if (part >= (int)gridDim.x)
          sumsq[row * 256 + part] = 0.f;
      }
  }

  // K split across workgroups (blockIdx.z = part).  Every workgroup leaves its sums in the workspace,
  // [part][block row][tile][row group][r * 64 + lane] floats, and takes a ticket; the workgroup that arrives last
  // adds the parts in part order (the same sums whichever workgroup that is) and runs the epilogue.  Nobody waits.
  // sumsq (MG == 1): the finishing workgroup also leaves the row sums of squares, see leave_row_sums().
  __device__ __forceinline__ void finish_split(const DecodeParams& p, const DecodeSeg& sg, f32x4 (&acc)[NACC][MG],
                                               float* red, int ltile0, int stride = ELEMS, float* sumsq = nullptr) {
    static_assert(!DUAL, "the gate/up pair is not split");
    __shared__ int arrived_last;
    settle();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int W = nwaves();
    float* mine = red + wave * stride;
#pragma unroll
    for (int a = 0; a < NACC; a++)
#pragma unroll
      for (int mg = 0; mg < MG; mg++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          mine[(a * MG + mg) * 256 + r * 64 + lane] = acc[a][mg][r];
    __syncthreads();
    const size_t part_stride = (size_t)gridDim.y * p.total_tiles * (MG * 256);
    float* part = p.part + ((size_t)blockIdx.y * p.total_tiles + sg.tile0 + ltile0) * (MG * 256);
    float own[MAXE];
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      const int e = threadIdx.x + i * nthreads();
      own[i] = 0.f;
      if (e < OUT) {
#pragma unroll
        for (int w = 0; w < (FIXW ? FIXW : W); w++)
          own[i] += red[w * stride + e];
        if (ltile0 + e / (MG * 256) < sg.tiles)
          __hip_atomic_store(part + blockIdx.z * part_stride + e, own[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    // The sums travel as device-scope atomic stores and loads (written through to, and read from, the level all
    // XCDs share), so no cache write-back or invalidate is needed: a device-wide fence here costs more than the
    // whole kernel (measured: +8 us with one fencing thread per workgroup, +40 us with all).  Order: every thread
    // waits until its own stores have been acknowledged (vmcnt counts stores on this target, and a workgroup
    // barrier by itself does NOT wait for the global stores of the other waves), then the barrier, then the
    // ticket, then the loads.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      const unsigned int last = (unsigned int)p.S - 1;
      arrived_last = atomicInc(&sk_split_tickets[p.ticket0 + blockIdx.y * gridDim.x + blockIdx.x], last) == last;
    }
    __syncthreads();
    if (!arrived_last)
      return;
    float pv[MAXE][4];
#pragma unroll
    for (int i = 0; i < MAXE; i++)
#pragma unroll
      for (int k = 0; k < 4; k++) {
        pv[i][k] = 0.f;
        if (off[i] >= 0 && k < p.S && k != (int)blockIdx.z)
          pv[i][k] = __hip_atomic_load(part + k * part_stride + threadIdx.x + i * nthreads(), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
      }
    float ov[MAXE];
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      ov[i] = 0.f;
      if (off[i] >= 0) {
        float v = 0.f;
#pragma unroll
        for (int k = 0; k < 4; k++)
          if (k < p.S)
            v += k == (int)blockIdx.z ? own[i] : pv[i][k];
        const uint32_t out = apply_post_bits(v + bf16_bits_to_f32(bias[i]), sg.post_op, in1[i], in2[i], sg.post_scale);
        sg.y[off[i]] = (uint16_t)out;
        ov[i] = bf16_bits_to_f32(out & 0xffffu);
      }
    }
    if (MG == 1 && sumsq) // uniform
      leave_row_sums(ov, sumsq, p.M);
  }

  // stride = floats between the regions of two waves (>= ELEMS).  sumsq (MG == 1, not the gate/up pair): also
  // leave, per row, the sum of squares of this workgroup's rounded outputs in sumsq[row][blockIdx.x] of a
  // [16][256] table (workgroup 0 zeroes the slots past the grid), added in a fixed order.
  __device__ __forceinline__ void finish(const DecodeSeg& sg, f32x4 (&acc)[NACC][MG], float* red, int stride = ELEMS,
                                         float* sumsq = nullptr, int M = 0) {
    settle();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int W = nwaves();
    float* mine = red + wave * stride;
#pragma unroll
    for (int a = 0; a < NACC; a++)
#pragma unroll
      for (int mg = 0; mg < MG; mg++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          mine[(a * MG + mg) * 256 + r * 64 + lane] = acc[a][mg][r];
    __syncthreads();
    // (no branch per output: slots past the outputs repeat the last one and are not stored, so the outputs' LDS reads
    // and post-op chains interleave)
    float v[MAXE], v2[MAXE];
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      const int e = min((int)threadIdx.x + i * nthreads(), OUT - 1);
      v[i] = v2[i] = 0.f;
#pragma unroll
      for (int w = 0; w < (FIXW ? FIXW : W); w++)
        v[i] += red[w * stride + e];
      if (DUAL) {
#pragma unroll
        for (int w = 0; w < (FIXW ? FIXW : W); w++)
          v2[i] += red[w * stride + e + ELEMS / 2];
      }
    }
    uint32_t out[MAXE];
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      if (DUAL) {
        const uint32_t gact = apply_post_bits(v[i] + bf16_bits_to_f32(bias[i]), TPPX_POST_SILU, 0, 0, 1.0f);
        out[i] = apply_post_bits(v2[i] + bf16_bits_to_f32(bias2[i]), TPPX_POST_MUL, gact, 0, 1.0f);
      } else {
        out[i] = apply_post_bits(v[i] + bf16_bits_to_f32(bias[i]), sg.post_op, in1[i], in2[i], sg.post_scale);
      }
    }
    float ov[MAXE];
#pragma unroll
    for (int i = 0; i < MAXE; i++) {
      ov[i] = 0.f;
      if (off[i] >= 0) {
        sg.y[off[i]] = (uint16_t)out[i];
        ov[i] = bf16_bits_to_f32(out[i] & 0xffffu);
      }
    }
    if (!DUAL && MG == 1 && sumsq) // uniform
      leave_row_sums(ov, sumsq, M);
  }
};

// ---------------------------------------------------------------------------
// QINT8 (W8A8), activations already quantised (int8 [M][K] + f32 [M][K/qbs]).
// ---------------------------------------------------------------------------
template <int MG, int NTW, int PF, int MAXW, int MINW, bool XOP>
__global__ void __launch_bounds__(MAXW * 64)
skinny_qint8_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int MPAD = MG * 16;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int W = MAXW == MINW ? MAXW : (int)(blockDim.x >> 6); // (a constant where it can be: divisions become shifts)
  const int grp = blockIdx.x;
  const DecodeSeg& sg = p.seg[sk_find_seg(p, grp)];
  const int ltile0 = (grp - sg.grp0) * NTW;
  const int m0 = blockIdx.y * MPAD;
  const int NB = p.nblk, TPB = p.tpb, KT = NB * TPB, G = p.deal;
  // K is dealt in runs of G tiles.  G == 4 (a scale block is a whole number of 256-wide runs; one run by default):
  // static ring slots, the int32 sums are folded after every run with the scales of the run's block.
  const bool FAST = G == 4;
  constexpr int UN = (PF % 4 == 0) ? PF : (PF % 2 == 0 ? 2 * PF : 4 * PF); // lcm(PF, 4) tiles per unrolled trip
  // runs of this workgroup (all of them unless K is split across workgroups), then of this wave
  const int ub = sk_share_pow2(blockIdx.z, p.units, p.S), ue = sk_share_pow2(blockIdx.z + 1, p.units, p.S);
  const int u0 = ub + sk_share(wave, ue - ub, W), u1 = ub + sk_share(wave + 1, ue - ub, W);
  const int t0 = u0 * G, t1 = u1 * G;
  const unsigned int magic = p.tpb_magic;
  auto blk_of = [&](int t) { // scale block of tile t (uniform): t / TPB without the division
    return magic ? (int)__umulhi((unsigned int)t, magic) : t;
  };
  const int b0 = blk_of(max(min(t0, KT - 1), 0)); // first scale block of this wave

  const i32x4* wq[NTW];
  const float* ws[NTW];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++) {
    const int64_t lt = min(ltile0 + nt, sg.tiles - 1); // ragged last group: duplicate, not stored
    wq[nt] = reinterpret_cast<const i32x4*>(sg.qw) + lt * KT * 64 + lane;
    ws[nt] = reinterpret_cast<const float*>(sg.sw) + lt * NB * 16 + (lane & 15);
  }
  // XOP: activations in operand order, one contiguous 1 KiB read per (k-tile,
  // row tile); otherwise row-major rows, 16 rows x 64 B per read.
  const int8_t* xrow[MG];
  const i32x4* xop = reinterpret_cast<const i32x4*>(p.xq) + (int64_t)blockIdx.y * MG * 64 + lane;
  const int xstride = p.mt * 64;
#pragma unroll
  for (int mg = 0; mg < MG; mg++) {
    const int m = min(m0 + mg * 16 + (lane & 15), p.M - 1);
    xrow[mg] = reinterpret_cast<const int8_t*>(p.xq) + (int64_t)m * p.K + (lane >> 4) * 16;
  }

  float* red = sk_lds;
  float* sa_s = sk_lds + (size_t)W * NTW * MG * 256 + (size_t)wave * p.cht * MPAD;
  const int nsa = t0 < t1 ? (blk_of(t1 - 1) - b0 + 1) * MPAD : 0;
  const int mtp = p.mt * 16;
  constexpr int SAB = 2 * MG; // loads per batch: 8 K blocks of this wave
  auto load_sa = [&](int i) {
    i = max(min(i, nsa - 1), 0);
    const int ul = i / MPAD, mr = i - ul * MPAD;
    // XOP: scales transposed by the quantisation kernel, [K/qbs][mt*16]
    return XOP ? p.sa[(int64_t)(b0 + ul) * mtp + m0 + mr] : p.sa[(int64_t)min(m0 + mr, p.M - 1) * NB + b0 + ul];
  };

  // Ring of PF stages; a stage = the weight tiles, their block scale and the
  // activation operand of one k-tile.  The main loop has NO branch and NO load
  // other than the ring itself, so the compiler's wait counts stay exact and
  // PF stages are really in flight (a load that must be waited for out of
  // order, or a branch inside the loop, drains the whole ring).
  i32x4 wreg[PF][NTW], xreg[PF][MG];
  float sreg[PF][NTW];
  auto load_stage = [&](int st, int t) {
    t = max(min(t, t1 - 1), 0); // past the end: re-read the last tile (never consumed)
    const int b = blk_of(t);
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      wreg[st][nt] = __builtin_nontemporal_load(wq[nt] + (int64_t)t * 64);
      sreg[st][nt] = ws[nt][b * 16];
    }
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      xreg[st][mg] = XOP ? xop[(int64_t)t * xstride + mg * 64] : *reinterpret_cast<const i32x4*>(xrow[mg] + t * 64);
  };
  // The ring's first requests are the kernel's first vector loads: the set-up of the epilogue (offsets and post-op
  // inputs of up to six outputs per thread) is several hundred instructions, which two waves per SIMD take 2 us to
  // get through.  (Timestamps: with the ring in front, a wave's first request goes out 0.8 instead of 2.1 us after
  // the first wave's start -- and its first tile still arrives about 4 us after the start: the memory system's own
  // start-up, not the request time, sets the beginning of the stream, so the kernel's time did not change.)  Loads
  // return in issue order, so the activation scales (L2) wait for the first stages; they are needed after four tiles.
  // (no branch around these first requests: behind a conditional load the compiler can no longer count the loads
  // in flight and waits for all of them; a wave without K blocks re-reads valid data it never uses)
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_stage(i, t0 + i);
  __builtin_amdgcn_sched_barrier(0); // keep the issue order of independent loads (see skinny_qint8_fq_kernel)
  // activation scales of this wave's K blocks, transposed in LDS: [u - u0][MPAD]
  float sa0[SAB];
#pragma unroll
  for (int j = 0; j < SAB; j++)
    sa0[j] = load_sa(j * 64 + lane);
  __builtin_amdgcn_sched_barrier(0);
  SkEpilogue<MG, NTW, false, MINW, (MAXW == MINW ? MAXW : 0)> ep;
  ep.prefetch_flat(p, sg, ltile0, m0);
  __builtin_amdgcn_sched_barrier(0);
  if (t0 < t1) {
    // the scales were requested first, so they are here long before the ring
#pragma unroll
    for (int j = 0; j < SAB; j++)
      if (j * 64 + lane < nsa)
        sa_s[j * 64 + lane] = sa0[j];
    for (int i0 = SAB * 64; i0 < nsa; i0 += SAB * 64) { // more than 8 K blocks per wave: rare
      float v[SAB];
#pragma unroll
      for (int j = 0; j < SAB; j++)
        v[j] = load_sa(i0 + j * 64 + lane);
#pragma unroll
      for (int j = 0; j < SAB; j++)
        if (i0 + j * 64 + lane < nsa)
          sa_s[i0 + j * 64 + lane] = v[j];
    }
  }

  f32x4 facc[NTW][MG];
  i32x4 iacc[NTW][MG];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++) {
      facc[nt][mg] = f32x4{0.f, 0.f, 0.f, 0.f};
      iacc[nt][mg] = i32x4{0, 0, 0, 0};
    }

  // multiply stage i (tile tt); `last` = tt closes a K block or this wave's part of one: fold into fp32
  auto consume = [&](int i, int tt, bool last) {
    float swv[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      swv[nt] = sreg[i][nt];
#pragma unroll
      for (int mg = 0; mg < MG; mg++)
        iacc[nt][mg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xreg[i][mg], wreg[i][nt], iacc[nt][mg], 0, 0, 0);
    }
    if (last) {
      const int b = blk_of(tt);
#pragma unroll
      for (int mg = 0; mg < MG; mg++) {
        const f32x4 sav = *reinterpret_cast<const f32x4*>(sa_s + (b - b0) * MPAD + mg * 16 + (lane >> 4) * 4);
#pragma unroll
        for (int nt = 0; nt < NTW; nt++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            facc[nt][mg][r] = fmaf((float)iacc[nt][mg][r], sav[r] * swv[nt], facc[nt][mg][r]);
            iacc[nt][mg][r] = 0;
          }
      }
    }
  };

  int t = t0;
  if (FAST) {
    // full trips of UN tiles: static ring slots and fold points (t0 is a
    // multiple of 4), every reload a real tile
    for (; t + UN + PF <= t1; t += UN) {
#pragma unroll
      for (int i = 0; i < UN; i++) {
        consume(i % PF, t + i, (i & 3) == 3);
        load_stage(i % PF, t + i + PF);
        __builtin_amdgcn_sched_barrier(0); // keep the reload right behind its stage: the ring stays PF deep
      }
    }
  }
  // remaining tiles (and every tile when K is not dealt in runs of 4 tiles);
  // the ring slot of tile tt is (tt - t0) % PF
  for (int tb = t; tb < t1; tb += PF) {
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int tt = tb + i;
      if (tt < t1) {
        consume(i, tt, FAST ? (tt & 3) == 3 : ((tt + 1) % TPB == 0 || tt + 1 == t1));
        if (tt + PF < t1)
          load_stage(i, tt + PF);
      }
    }
  }
  if (p.S > 1)
    ep.finish_split(p, sg, facc, red, ltile0);
  else
    ep.finish(sg, facc, red);
}

// ---------------------------------------------------------------------------
// QINT8, 17..64 rows, few channel tiles and a long K (the Llama down-projection): in the kernel above every wave
// pulls its own activation operands, so a workgroup drags M x K bytes of int8 activations through its CU beside
// 1-2 tiles' worth of weights, and the CU's load path, not HBM, sets the pace.  Here the sixteen waves form a
// TW x KPW grid: wave (tw, kp) owns channel tile tw over K part kp of the workgroup's K slice, and the TW waves of a
// K part share the activation operands of each 256-wide run through LDS (each fetches 1 / TW of the run's 4 x MG
// operand tiles; one barrier per run).  With K split over S workgroups that own TW tiles each, the grid still fills
// the chip and a workgroup reads 1 / (TW * S) of the activations per weight tile it streams.
// Workgroup id -> (channel group id / S, K slice id % S): the workgroups of one XCD (ids equal mod 8) then share ONE
// K slice when S divides 8, so every XCD's L2 fetches only that slice of the activations from memory.
// The K slices' partial tiles travel as 128-bit device-scope stores and loads (16 bytes per lane instruction; as
// dwords the exchange cost more than the split saved), merged by the last workgroup to arrive, in slice order.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void sk_store_x4_device(float* dst, f32x4 v) {
  // device scope: performed where every XCD observes it (the 128-bit form of the atomic stores of finish_split)
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
}
__device__ __forceinline__ f32x4 sk_load_x4_device(const float* src) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(src) : "memory");
  return v;
}

// Epilogue of the TW x KPW kernels: the K parts' sums meet in LDS, the K slices' partial tiles in the workspace
// (128-bit device-scope stores / loads, arrival counter as in SkEpilogue::finish_split), then bias, rounding and
// post-op.  Thread t finishes Q quads of four adjacent channels of one row, e = (q * W * 64 + t) * 4 .., of the
// workgroup's outputs e = ((tw * MG + mg) * 4 + r) * 64 + lane.  Called by every thread, after the main loop.
// TPW = channel tiles per wave (tw = the wave's first tile); the workgroup has (TW / TPW) * KPW waves.
template <int MG, int TW, int KPW, int TPW = 1>
__device__ __forceinline__ void sk_nk_finish(const DecodeParams& p, const DecodeSeg& sg, f32x4 (&facc)[TPW][MG], float* sk_lds,
                                             int grp, int z, int tw, int kp, int ltile0, int m0) {
  constexpr int W = (TW / TPW) * KPW;
  constexpr int OUT = TW * MG * 256;
  const int lane = threadIdx.x & 63;
  const int S = p.S;
  constexpr int Q = (OUT + W * 256 - 1) / (W * 256);
  int64_t o[Q];
  bool valid[Q];
  uint2 bias2[Q], in1[Q], in2[Q];
#pragma unroll
  for (int q = 0; q < Q; q++) {
    const int e0 = (q * W * 64 + (int)threadIdx.x) * 4;
    const int el = e0 & 63, er = (e0 >> 6) & 3, emg = (e0 >> 8) % MG, etw = (e0 >> 8) / MG;
    const int m = m0 + emg * 16 + (el >> 4) * 4 + er;
    const int n = (ltile0 + etw) * 16 + (el & 15);
    valid[q] = e0 < OUT && m < p.M && (ltile0 + etw) < sg.tiles;
    o[q] = (int64_t)m * sg.N + n;
    bias2[q] = in1[q] = in2[q] = make_uint2(0, 0);
    if (valid[q]) { // requested now, used after the reduction (and, with a K split, after the arrival counter)
      if (sg.bias)
        bias2[q] = *reinterpret_cast<const uint2*>(sg.bias + n);
      if (sg.post_in)
        in1[q] = *reinterpret_cast<const uint2*>(sg.post_in + o[q]);
      if (sg.post_in2)
        in2[q] = *reinterpret_cast<const uint2*>(sg.post_in2 + o[q]);
    }
  }
  __syncthreads(); // everybody has read the last operands: the scratch takes their place
  float* red = sk_lds; // [kp][OUT]
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
#pragma unroll
      for (int r = 0; r < 4; r++)
        red[(size_t)kp * OUT + (((tw + t) * MG + mg) * 4 + r) * 64 + lane] = facc[t][mg][r];
  __syncthreads();
  f32x4 own[Q], tot[Q];
#pragma unroll
  for (int q = 0; q < Q; q++) {
    const int e0 = min((q * W * 64 + (int)threadIdx.x) * 4, OUT - 4); // threads past the outputs repeat the last quad
    own[q] = *reinterpret_cast<const f32x4*>(red + e0);
#pragma unroll
    for (int k = 1; k < KPW; k++)
      own[q] += *reinterpret_cast<const f32x4*>(red + (size_t)k * OUT + e0);
    tot[q] = own[q];
  }
  if (S > 1) {
    __shared__ int arrived_last;
    // partial tiles [slice][block row][channel group][OUT]: whole groups, so a ragged last group stays inside its slot
    const size_t slice_stride = (size_t)gridDim.y * (gridDim.x / S) * OUT;
    // (threads past the outputs write and read the last quad again: the same values)
    float* mine = p.part + ((size_t)blockIdx.y * (gridDim.x / S) + grp) * OUT +
                  (size_t)min((int)threadIdx.x * 4, OUT - 4 - (Q - 1) * W * 256);
#pragma unroll
    for (int q = 0; q < Q; q++)
      sk_store_x4_device(mine + (size_t)z * slice_stride + q * W * 256, own[q]);
    // every thread's stores acknowledged at device scope, then the barrier, then the ticket, then the loads (see
    // SkEpilogue::finish_split)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      const unsigned int last = (unsigned int)S - 1;
      arrived_last = atomicInc(&sk_split_tickets[p.ticket0 + blockIdx.y * (gridDim.x / S) + grp], last) == last;
    }
    __syncthreads();
    if (!arrived_last)
      return;
#pragma unroll
    for (int q = 0; q < Q; q++) {
      f32x4 other[4];
#pragma unroll
      for (int k = 0; k < 4; k++)
        other[k] = (k < S && k != z) ? sk_load_x4_device(mine + (size_t)k * slice_stride + q * W * 256) : f32x4{0.f, 0.f, 0.f, 0.f};
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(other[0]), "+v"(other[1]), "+v"(other[2]), "+v"(other[3])::"memory");
      tot[q] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < 4; k++)
        if (k < S)
          tot[q] += (k == z) ? own[q] : other[k]; // slice order: the same sums whichever workgroup arrives last
    }
  }
  // (no branch per quad around the arithmetic: the quads' post-op chains interleave; only the store is conditional)
  uint32_t out[Q][2];
#pragma unroll
  for (int q = 0; q < Q; q++) {
    const uint32_t bw[2] = {bias2[q].x, bias2[q].y}, w1[2] = {in1[q].x, in1[q].y}, w2[2] = {in2[q].x, in2[q].y};
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const uint32_t a = apply_post_bits(tot[q][2 * h] + bf16_bits_to_f32(bw[h] & 0xffffu), sg.post_op, w1[h] & 0xffffu,
                                         w2[h] & 0xffffu, sg.post_scale);
      const uint32_t b = apply_post_bits(tot[q][2 * h + 1] + bf16_bits_to_f32(bw[h] >> 16), sg.post_op, w1[h] >> 16,
                                         w2[h] >> 16, sg.post_scale);
      out[q][h] = (a & 0xffffu) | (b << 16);
    }
  }
#pragma unroll
  for (int q = 0; q < Q; q++)
    if (valid[q])
      *reinterpret_cast<uint2*>(sg.y + o[q]) = make_uint2(out[q][0], out[q][1]);
}

template <int MG, int TW, int KPW, int WPF, int XPF, int MAXSTEPS>
__global__ void __launch_bounds__(TW * KPW * 64)
skinny_qint8_nk_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int W = TW * KPW;
  constexpr int XT = 4 * MG;              // operand tiles per run: tile j = k-tile j / MG, row group j % MG
  constexpr int XPW = (XT + TW - 1) / TW; // fetched by one wave: j = tw + TW * i
  constexpr int OUT = TW * MG * 256;      // outputs of the workgroup, element e = ((tw * MG + mg) * 4 + r) * 64 + lane
  static_assert(XPF <= WPF, "the weights (HBM) are requested at least as far ahead as the activations (L2)");
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tw = wave % TW, kp = wave / TW;
  const int S = p.S;
  const int grp = (int)blockIdx.x / S, z = (int)blockIdx.x % S;
  const DecodeSeg& sg = p.seg[0];
  const int ltile0 = grp * TW;
  const int m0 = blockIdx.y * (MG * 16);
  const int NR = p.units, NB = p.nblk; // 256-wide runs of K, scale blocks
  const unsigned int magic = p.spb_magic;
  auto blk_of_run = [&](int u) { return magic ? (int)__umulhi((unsigned int)u, magic) : u; };
  // runs of this workgroup's K slice, then of this wave's K part; every wave makes the same number of steps
  const int ub = sk_share_pow2(z, NR, S), ue = sk_share_pow2(z + 1, NR, S);
  const int u0 = ub + (kp * (ue - ub)) / KPW, u1 = ub + ((kp + 1) * (ue - ub)) / KPW;
  const int nsteps = (ue - ub + KPW - 1) / KPW; // <= MAXSTEPS (the launcher checks)

  const int64_t lt = min(ltile0 + tw, sg.tiles - 1); // ragged last group: duplicate, not stored
  const i32x4* wq = reinterpret_cast<const i32x4*>(sg.qw) + lt * ((int64_t)NR * 4) * 64 + lane;
  const float* ws = reinterpret_cast<const float*>(sg.sw) + lt * NB * 16 + (lane & 15);
  const i32x4* xop = reinterpret_cast<const i32x4*>(p.xq) + (int64_t)blockIdx.y * MG * 64 + lane;
  const int xstride = p.mt * 64, mtp = p.mt * 16;

  // Two rings: weights (from HBM) WPF steps ahead, the wave's share of the activation operands and the scales
  // (L2-resident) XPF steps ahead.  Loads return in issue order, so a step's activations are requested BEFORE
  // weights of later steps wherever both are issued together.
  i32x4 wreg[WPF][4], xreg[XPF][XPW];
  float sreg[XPF], sareg[XPF];
  auto run_of = [&](int s) { return min(min(u0 + s, max(u1 - 1, u0)), NR - 1); }; // past the part's end: re-read (never used)
  auto load_w = [&](int st, int s) {
    const int u = run_of(s);
#pragma unroll
    for (int kt = 0; kt < 4; kt++)
      wreg[st][kt] = __builtin_nontemporal_load(wq + (int64_t)(u * 4 + kt) * 64);
  };
  auto load_x = [&](int st, int s) {
    const int u = run_of(s), b = blk_of_run(u);
#pragma unroll
    for (int i = 0; i < XPW; i++) {
      const int j = min(tw + TW * i, XT - 1);
      xreg[st][i] = xop[(int64_t)(u * 4 + j / MG) * xstride + (j % MG) * 64];
    }
    sreg[st] = ws[b * 16];
    // activation scales of the run's block, transposed by the quantisation kernel: [K block][mt * 16 rows]
    sareg[st] = p.sa[(int64_t)b * mtp + m0 + min(lane, MG * 16 - 1)];
  };
  static_for<0, WPF>([&](auto I) {
    constexpr int i = decltype(I)::value;
    if constexpr (i < XPF)
      load_x(i, i);
    load_w(i, i);
  });

  // LDS: operand stage [buffer][K part][tile j][lane] x 16 B, then scales [buffer][K part][64]; the reduction of the
  // epilogue reuses the space
  i32x4* xs = reinterpret_cast<i32x4*>(sk_lds);
  float* sas = sk_lds + (size_t)2 * KPW * XT * 256;
  f32x4 facc[1][MG];
  i32x4 iacc[MG];
#pragma unroll
  for (int mg = 0; mg < MG; mg++) {
    facc[0][mg] = f32x4{0.f, 0.f, 0.f, 0.f};
    iacc[mg] = i32x4{0, 0, 0, 0};
  }
  static_for<0, MAXSTEPS>([&](auto SS) {
    constexpr int s = decltype(SS)::value;
    constexpr int wi = s % WPF, xi = s % XPF;
    if (s < nsteps) { // uniform over the workgroup
      i32x4* xb = xs + (size_t)(((s & 1) * KPW + kp) * XT) * 64 + lane;
      float* sb = sas + ((s & 1) * KPW + kp) * 64;
#pragma unroll
      for (int ii = 0; ii < XPW; ii++)
        if (tw + TW * ii < XT)
          xb[(tw + TW * ii) * 64] = xreg[xi][ii];
      if (tw == 0)
        sb[lane] = sareg[xi];
      const float swv = sreg[xi];
      if (s + XPF < nsteps)
        load_x(xi, s + XPF);
      // one barrier per step: a wave that reaches the barrier of step s + 1 has finished reading the stage of
      // step s, so that buffer may be overwritten for step s + 2
      __syncthreads();
      if (u0 + s < u1) {
#pragma unroll
        for (int kt = 0; kt < 4; kt++)
#pragma unroll
          for (int mg = 0; mg < MG; mg++)
            iacc[mg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xb[(kt * MG + mg) * 64], wreg[wi][kt], iacc[mg], 0, 0, 0);
#pragma unroll
        for (int mg = 0; mg < MG; mg++) {
          const f32x4 sav = *reinterpret_cast<const f32x4*>(sb + mg * 16 + (lane >> 4) * 4);
#pragma unroll
          for (int r = 0; r < 4; r++) {
            facc[0][mg][r] = fmaf((float)iacc[mg][r], sav[r] * swv, facc[0][mg][r]);
            iacc[mg][r] = 0;
          }
        }
      }
      if (s + WPF < nsteps)
        load_w(wi, s + WPF);
    }
  });

  sk_nk_finish<MG, TW, KPW, 1>(p, sg, facc, sk_lds, grp, z, tw, kp, ltile0, m0);
}

// ---------------------------------------------------------------------------
// MXFP4, 33..64 rows, few channel tiles and a long K: the same TW x KPW grid of waves.  Wave (tw, kp) owns channel
// tile tw over K part kp of the workgroup's K slice; per K tile (128 channels) the TW = MG waves of a K part stage
// the 64 x 128 bf16 activations in LDS once -- wave tw fetches row group tw with row-contiguous 16-byte loads and
// writes it in the swizzled operand-order image of skinny_mxfp4_mg_kernel -- and every wave reads all of it as MFMA
// operands.  Against that kernel, where each wave stages the whole tile for itself, a workgroup moves a quarter of
// the activation bytes per weight tile, and a wave's whole weight range (one 1 KiB tile per step) is in flight from
// the first instruction.  K slices across workgroups and the merge as in skinny_qint8_nk_kernel.
// ---------------------------------------------------------------------------
template <int MG, int TW, int TPW, int KPW, int WPF, int XPF, int MAXSTEPS>
__global__ void __launch_bounds__((TW / TPW) * KPW * 64)
skinny_mxfp4_nk_kernel(const DecodeParams p) {
  constexpr int WC = TW / TPW;  // wave columns: wave (wc, kp) owns channel tiles wc*TPW .. of K part kp
  constexpr int RGW = MG / WC;  // row groups of a K tile's activations that one wave stages
  static_assert(WC * TPW == TW && RGW * WC == MG, "tiles and row groups divide among the wave columns");
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int MPAD = MG * 16, XI = RGW * 4; // items (4 rows x 256 B) a wave stages per K tile
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wc = wave % WC, kp = wave / WC;
  const int S = p.S;
  const int grp = (int)blockIdx.x / S, z = (int)blockIdx.x % S;
  const DecodeSeg& sg = p.seg[0];
  const int ltile0 = grp * TW;
  const int m0 = blockIdx.y * MPAD;
  const int KT = p.units; // K tiles of 128
  const int tb = sk_share(z, KT, S), te = sk_share(z + 1, KT, S);
  const int t0 = tb + (kp * (te - tb)) / KPW, t1 = tb + ((kp + 1) * (te - tb)) / KPW;
  const int nsteps = (te - tb + KPW - 1) / KPW; // <= MAXSTEPS (the launcher checks)

  uint32_t woff[TPW];
#pragma unroll
  for (int t = 0; t < TPW; t++)
    woff[t] = (uint32_t)(min(ltile0 + wc * TPW + t, sg.tiles - 1) * KT * 64 + lane);
  const char* qwb = reinterpret_cast<const char*>(sg.qw);
  const char* swb = reinterpret_cast<const char*>(sg.sw);
  const char* xb = reinterpret_cast<const char*>(p.x);
  const int r4 = lane >> 4, c16 = lane & 15;
  // Every workgroup of a K slice reads the same activation tiles; walking them in the same order, all of them ask
  // the same L2 channels for the same lines at the same moment.  Workgroup `grp` starts `grp` tiles into its part
  // and wraps round: the sums are added in a rotated (fixed) order.
  const int len = t1 - t0, rot = len > 0 ? grp % len : 0;
  auto tile_of = [&](int s) { // past the part's end: a valid tile, never consumed
    const int i = s + rot;
    return max(min(t0 + (i >= len ? i - len : i), t1 - 1), 0);
  };

  i32x4 wreg[WPF][TPW], xr[XPF][XI];
  uint32_t sreg[WPF][TPW];
  auto load_w = [&](int st, int s) {
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      const uint32_t slot = woff[t] + (uint32_t)tile_of(s) * 64u;
      wreg[st][t] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(qwb + (size_t)(slot * 16u)));
      sreg[st][t] = *reinterpret_cast<const uint8_t*>(swb + (size_t)slot);
    }
  };
  // this wave's share of a K tile's activations: rows wc*RGW*16 + it*4 + lane/16, chunk lane%16 of the tile's 256
  // bytes; rows past M re-read row M-1 (their results are not stored)
  auto load_x = [&](int st, int s) {
    const uint32_t base = (uint32_t)tile_of(s) * 256u + (uint32_t)c16 * 16u;
#pragma unroll
    for (int it = 0; it < XI; it++) {
      const int row = min(m0 + wc * (RGW * 16) + it * 4 + r4, p.M - 1);
      xr[st][it] = *reinterpret_cast<const i32x4*>(xb + (size_t)((uint32_t)(row * p.K) * 2u + base));
    }
  };
  // a step's activations are requested before weights of later steps (loads return in issue order)
  static_for<0, WPF>([&](auto I) {
    constexpr int i = decltype(I)::value;
    if constexpr (i < XPF)
      load_x(i, i);
    load_w(i, i);
  });

  // LDS: [buffer][K part][chunk 16][row MPAD] x 16 B; the reduction of the epilogue reuses the space
  i32x4* xs = reinterpret_cast<i32x4*>(sk_lds);
  int rdo[4]; // operand slot of this lane for step j: chunk g*4 + j, row m of row group mg (+ mg*16)
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int cj = (lane >> 4) * 4 + j;
    rdo[j] = cj * MPAD + ((lane & 15) ^ cj);
  }
  f32x4 acc[TPW][MG];
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      acc[t][mg] = f32x4{0.f, 0.f, 0.f, 0.f};

  static_for<0, MAXSTEPS>([&](auto SS) {
    constexpr int s = decltype(SS)::value;
    constexpr int wi = s % WPF, xi = s % XPF;
    if (s < nsteps) { // uniform over the workgroup
      i32x4* stage = xs + (size_t)((s & 1) * KPW + kp) * (MPAD * 16);
#pragma unroll
      for (int it = 0; it < XI; it++)
        stage[c16 * MPAD + ((wc * (RGW * 16) + it * 4 + r4) ^ c16)] = xr[xi][it];
      if (s + XPF < nsteps)
        load_x(xi, s + XPF);
      // one barrier per step: a wave that reaches the barrier of step s + 1 has finished reading the stage of
      // step s, so that buffer may be overwritten for step s + 2
      __syncthreads();
      if (t0 + s < t1) {
        float sc[TPW];
#pragma unroll
        for (int t = 0; t < TPW; t++)
          sc[t] = e8m0_to_f32(sreg[wi][t]);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          bf16x8 b[TPW];
#pragma unroll
          for (int t = 0; t < TPW; t++)
            b[t] = sk_cvt_fp4x8((uint32_t)wreg[wi][t][j], sc[t]);
#pragma unroll
          for (int mg = 0; mg < MG; mg++) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, stage[rdo[j] + mg * 16]);
#pragma unroll
            for (int t = 0; t < TPW; t++)
              acc[t][mg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[t], acc[t][mg], 0, 0, 0);
          }
        }
      }
      if (s + WPF < nsteps)
        load_w(wi, s + WPF);
    }
  });
  sk_nk_finish<MG, TW, KPW, TPW>(p, sg, acc, sk_lds, grp, z, wc * TPW, kp, ltile0, m0);
}

// ---------------------------------------------------------------------------
// QINT8 with the activation quantisation fused in, for M <= 16 (qbs == 256).
// Every wave quantises the rows of its own K range (one (row, block) item =
// 16 lanes x 16 values, DPP max reduction) into a wave-private LDS region that
// keeps only the M valid rows of each operand tile, then reads its MFMA
// operand from there (lanes of the padded rows re-read row M-1), so the main
// loop issues weight loads only and the whole ring is in flight from the
// first instruction.
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float sk_dpp_max(float v) {
  int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
  return fmaxf(v, __int_as_float(o));
}
__device__ __forceinline__ float sk_wave_max(float v) {
  v = sk_dpp_max<0xB1>(v);  // quad_perm [1,0,3,2]
  v = sk_dpp_max<0x4E>(v);  // quad_perm [2,3,0,1]
  v = sk_dpp_max<0x141>(v); // row_half_mirror
  v = sk_dpp_max<0x140>(v); // row_mirror
  float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ int sk_int8_rne(float v, float inv) {
  float r = rintf(__fmul_rn(v, inv));
  return (int)fminf(fmaxf(r, -127.0f), 127.0f);
}

// Four values * inv, rounded to nearest even, as packed int8.  |v * inv| <= 127 up to rounding (inv = 1 / (amax / 127)
// or 0), so no clamp is needed; adding 1.5 * 2^23 to the rounded product rounds it to an integer exactly as rintf does
// and leaves its two's complement in the low mantissa byte.
__device__ __forceinline__ uint32_t sk_int8x4_rne(float a, float b, float c, float d, float inv) {
  const float magic = 12582912.0f;
  // the products must be rounded to f32 before the add (a fused multiply-add rounds once and differs in rare
  // cases); the empty asm makes each product opaque so that it cannot be contracted into the add
  float pa = a * inv, pb = b * inv, pc = c * inv, pd = d * inv;
  asm("" : "+v"(pa), "+v"(pb), "+v"(pc), "+v"(pd));
  const uint32_t ua = __float_as_uint(pa + magic), ub = __float_as_uint(pb + magic);
  const uint32_t uc = __float_as_uint(pc + magic), ud = __float_as_uint(pd + magic);
  // v_perm_b32: selector bytes 0..3 pick from the second operand, 4..7 from the first, 0x0c gives zero
  return __builtin_amdgcn_perm(ub, ua, 0x0c0c0400u) | __builtin_amdgcn_perm(ud, uc, 0x04000c0cu);
}

// BIGB: scale blocks of several 256-wide runs.  Every wave takes the maxima of its own (row, run) items, the waves
// exchange them through LDS (one barrier), and an item is quantised with the maximum over the runs of its block; all
// of a wave's items stay in registers meanwhile (the launcher checks that there are at most 4 * XB).
// WBITS = 4 / 2: QINT4 / ternary QINT2 weights streamed at their own width.  A 16-byte load per lane then holds the
// lane's operands of G = 8 / WBITS consecutive K tiles (tppx_pack_qint_tiles), expanded in registers right in front
// of the MFMA, two instructions per operand dword: 4-bit codes as 16 x value (the nibble moved to the top of its
// byte), ternary codes as 64 x value (two's complement in two bits -- 0, 1, 3 = -1 -- moved to the top of their
// byte); the fold divides by 16 or 64, which is exact.  The ring's stages are such loads (PF of them).
template <int WBITS>
__device__ __forceinline__ i32x4 sk_expand_codes(i32x4 w, int g) {
  i32x4 o;
  if constexpr (WBITS == 4) {
#pragma unroll
    for (int j = 0; j < 4; j++)
      o[j] = (int)((g == 0 ? ((uint32_t)w[j] << 4) : (uint32_t)w[j]) & 0xF0F0F0F0u);
  } else {
    // dword g = K tile g; its byte i holds the codes of byte i of the four operand dwords j, two bits each
    const uint32_t pw = (uint32_t)(g == 0 ? w[0] : g == 1 ? w[1] : g == 2 ? w[2] : w[3]);
#pragma unroll
    for (int j = 0; j < 4; j++)
      o[j] = (int)((j == 3 ? pw : (pw << (6 - 2 * j))) & 0xC0C0C0C0u);
  }
  return o;
}

template <int NTW, int PF, int MAXW, int MINW, int XB, bool BIGB, int WBITS = 8>
__global__ void __launch_bounds__(MAXW * 64)
skinny_qint8_fq_kernel(const DecodeParams p) {
  constexpr int G = 8 / WBITS; // K tiles per 16-byte weight load of a lane
  static_assert(WBITS == 8 || !BIGB, "the packed formats run 256-wide blocks");
  extern __shared__ __align__(16) float sk_lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int W = MAXW == MINW ? MAXW : (int)(blockDim.x >> 6);
  const int grp = blockIdx.x;
  const DecodeSeg& sg = p.seg[sk_find_seg(p, grp)];
  const int ltile0 = (grp - sg.grp0) * NTW;
  const int M = p.M; // <= 16, one block row
  const int NR = p.units, KT = NR * 4, NB = p.nblk; // 256-wide runs of K, tiles, scale blocks
  const int u0 = sk_share(wave, NR, W), u1 = sk_share(wave + 1, NR, W);
  const int t0 = u0 * 4, t1 = u1 * 4;
  const unsigned int magic = p.spb_magic;
  auto blk_of_run = [&](int u) { return BIGB ? (int)__umulhi((unsigned int)u, magic) : u; };

  const i32x4* wq[NTW];
  const float* ws[NTW];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++) {
    const int64_t lt = min(ltile0 + nt, sg.tiles - 1);
    wq[nt] = reinterpret_cast<const i32x4*>(sg.qw) + lt * (KT / G) * 64 + lane;
    ws[nt] = reinterpret_cast<const float*>(sg.sw) + lt * NB * 16 + (lane & 15);
  }
  // Loads return in issue order, so everything small and L2-resident that the
  // wave needs early (its activation rows, the post-op inputs) is requested
  // BEFORE the weight ring: waiting for it then does not wait for HBM.
  // One (row, block) item = 256 values = 16 lanes x 16 values, so a wave
  // quantises four items per pass and the max reduction stays inside a DPP
  // row.  Items are numbered row-fastest; XB passes are in flight at a time.
  const uint16_t* xb = reinterpret_cast<const uint16_t*>(p.x);
  const int nitems = M * (u1 - u0);
  const uint32_t Mu = (uint32_t)M, mmagic = p.m_magic;
  auto run_of_item = [&](uint32_t it) { return mmagic ? __umulhi(it, mmagic) : it; }; // it / M without the division
  i32x4 raw[XB][2]; // first-class vectors: copies of the HIP struct type would keep the array in scratch
  auto load_pass = [&](auto PS, int base) {
    constexpr int ps = decltype(PS)::value;
    const uint32_t it = (uint32_t)min((base + ps) * 4 + (lane >> 4), max(nitems - 1, 0));
    const uint32_t ul = run_of_item(it), mr = it - ul * Mu;
    const i32x4* src = reinterpret_cast<const i32x4*>(xb + (int64_t)mr * p.K + (int64_t)(u0 + (int)ul) * 256 + (lane & 15) * 16);
    raw[ps][0] = src[0];
    raw[ps][1] = src[1];
  };
  static_for<0, XB>([&](auto PS) { load_pass(PS, 0); });
  // (the scheduler is free to move independent loads past one another: pinned, or it puts some of the activation
  // requests behind the weight ring and the quantisation waits for HBM)
  __builtin_amdgcn_sched_barrier(0);
  SkEpilogue<1, NTW, false, MINW, (MAXW == MINW ? MAXW : 0)> ep;
  ep.prefetch_flat(p, sg, ltile0, 0);
  __builtin_amdgcn_sched_barrier(0);

  // ring stage = weight tiles + their block scale (see skinny_qint8_kernel)
  i32x4 wreg[PF][NTW];
  float sreg[PF][NTW];
  // (WBITS < 8: `t` counts 16-byte loads = groups of G tiles; t0, t1 are multiples of 4, so of G)
  auto load_stage = [&](int st, int t) {
    t = max(min(t, t1 / G - 1), 0); // past the end (or a wave without K blocks): re-read a valid tile, never consumed
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      wreg[st][nt] = __builtin_nontemporal_load(wq[nt] + (int64_t)t * 64);
      sreg[st][nt] = ws[nt][blk_of_run((t * G) >> 2) * 16];
    }
  };
  // No branch around the ring's first requests: with one, the compiler can no longer count the loads behind the
  // activations and waits for the whole ring before it lets the quantisation start.
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_stage(i, t0 / G + i);
  __builtin_amdgcn_sched_barrier(0);

  // wave-private LDS: xq [tile][g][M rows][16 B], then sa [unit][16]; the region of the cross-wave reduction
  // comes first unless both do not fit side by side (they overlap then, with a barrier in between)
  float* red = sk_lds;
  uint8_t* mine = reinterpret_cast<uint8_t*>(sk_lds + (p.lds_overlap ? 0 : (size_t)W * NTW * 256)) + (size_t)wave * p.cht * (256 * M + 64);
  uint32_t* xq_s = reinterpret_cast<uint32_t*>(mine);
  float* sa_s = reinterpret_cast<float*>(mine + (size_t)p.cht * 256 * M);
  // maximum of |x| over the 256 values of the pass's item, in every lane of its DPP row
  auto item_amax = [&](auto PS) {
    constexpr int ps = decltype(PS)::value;
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const uint32_t wd = (uint32_t)raw[ps][j >> 2][j & 3];
      amax = fmaxf(amax, fmaxf(fabsf(bf16_bits_to_f32(wd & 0xffffu)), fabsf(bf16_bits_to_f32(wd >> 16))));
    }
    amax = sk_dpp_max<0xB1>(amax);  // quad_perm [1,0,3,2]
    amax = sk_dpp_max<0x4E>(amax);  // quad_perm [2,3,0,1]
    amax = sk_dpp_max<0x141>(amax); // row_half_mirror
    return sk_dpp_max<0x140>(amax); // row_mirror: every lane of the row holds the max
  };
  // BIGB: [row][run] maxima of all waves, behind every wave's private region
  float* amax_s = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(sk_lds + (p.lds_overlap ? 0 : (size_t)W * NTW * 256)) +
                                           (size_t)W * p.cht * (256 * M + 64));
  if (BIGB) {
    static_for<0, XB>([&](auto PS) {
      constexpr int ps = decltype(PS)::value;
      if (ps * 4 < nitems) { // wave-uniform
        const int it = ps * 4 + (lane >> 4);
        const uint32_t itc = (uint32_t)min(it, nitems - 1);
        const uint32_t ul = run_of_item(itc), mr = itc - ul * Mu;
        const float am = item_amax(PS);
        if (it < nitems && (lane & 15) == 0)
          amax_s[mr * NR + u0 + ul] = am;
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    __syncthreads();
    // the values are unpacked again behind the barrier: kept across it, the floats of all passes would spill
#pragma unroll
    for (int ps = 0; ps < XB; ps++)
      asm volatile("" : "+v"(raw[ps][0]), "+v"(raw[ps][1]));
  }
  auto quant_pass = [&](auto PS, int base) {
    constexpr int ps = decltype(PS)::value;
    if ((base + ps) * 4 < nitems) { // wave-uniform
      const int it = (base + ps) * 4 + (lane >> 4);
      const uint32_t itc = (uint32_t)min(it, nitems - 1);
      const uint32_t ul = run_of_item(itc), mr = itc - ul * Mu;
      float v[16];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const uint32_t wd = (uint32_t)raw[ps][j >> 2][j & 3];
        v[2 * j] = bf16_bits_to_f32(wd & 0xffffu);
        v[2 * j + 1] = bf16_bits_to_f32(wd >> 16);
      }
      float amax;
      if (BIGB) {
        // the item's block = runs [blk * spb, (blk + 1) * spb): the 16 lanes of the DPP row share them out
        const int spb = p.tpb >> 2, r0 = blk_of_run(u0 + (int)ul) * spb;
        amax = 0.0f;
        for (int j = lane & 15; j < spb; j += 16)
          amax = fmaxf(amax, amax_s[mr * NR + r0 + j]);
        amax = sk_dpp_max<0xB1>(amax);
        amax = sk_dpp_max<0x4E>(amax);
        amax = sk_dpp_max<0x141>(amax);
        amax = sk_dpp_max<0x140>(amax);
      } else {
        amax = item_amax(PS);
      }
      // == float(double(amax) / 127.0): amax is a bf16 value, so the
      // quotient cannot sit on a double-rounding boundary
      const float sc = __fdiv_rn(amax, 127.0f);
      const float inv = sc != 0.0f ? __frcp_rn(sc) : 0.0f;
      uint32_t pk[4];
#pragma unroll
      for (int d = 0; d < 4; d++)
        pk[d] = sk_int8x4_rne(v[4 * d], v[4 * d + 1], v[4 * d + 2], v[4 * d + 3], inv);
      if (it < nitems) {
        // values k = (lane&15)*16.. of the run: tile (lane&15)/4, K group (lane&15)%4
        const int tl = (int)ul * 4 + ((lane & 15) >> 2), g = lane & 3;
        reinterpret_cast<uint4*>(xq_s)[(tl * 4 + g) * M + (int)mr] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        if ((lane & 15) == 0)
          sa_s[ul * 16 + mr] = sc; // per run: the runs of one block hold the same scale
      }
    }
    if (BIGB)
      __builtin_amdgcn_sched_barrier(0); // one pass after the other: interleaved, their temporaries spill
  };
  static_for<0, XB>([&](auto PS) { quant_pass(PS, 0); });
  if (!BIGB)
    for (int base = XB; base * 4 < nitems; base += XB) { // more than 4 * XB items per wave
      static_for<0, XB>([&](auto PS) { load_pass(PS, base); });
      static_for<0, XB>([&](auto PS) { quant_pass(PS, base); });
    }
  const int xoff = ((lane >> 4) * M + min(lane & 15, M - 1)) * 4; // dword offset inside a tile

  f32x4 facc[NTW][1];
  i32x4 iacc[NTW];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++) {
    facc[nt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
    iacc[nt] = i32x4{0, 0, 0, 0};
  }
  auto consume = [&](int i, int tt, bool last) {
    const i32x4 xa = *reinterpret_cast<const i32x4*>(xq_s + (tt - t0) * 16 * M + xoff);
    float swv[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      swv[nt] = sreg[i][nt];
      iacc[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa, wreg[i][nt], iacc[nt], 0, 0, 0);
    }
    if (last) { // K block complete
      // result rows (lane>>4)*4 + r; scales of rows >= M are whatever the LDS held: those rows are not stored
      const f32x4 sav = *reinterpret_cast<const f32x4*>(sa_s + ((tt >> 2) - u0) * 16 + (lane >> 4) * 4); // by run
#pragma unroll
      for (int nt = 0; nt < NTW; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          facc[nt][0][r] = fmaf((float)iacc[nt][r], sav[r] * swv[nt], facc[nt][0][r]);
          iacc[nt][r] = 0;
        }
    }
  };
  if constexpr (WBITS == 8) {
    int t = t0;
    for (; t + 2 * PF <= t1; t += PF) { // branch-free full groups (PF is a multiple of 4): every reload is a real tile
#pragma unroll
      for (int i = 0; i < PF; i++) {
        consume(i, t + i, (i & 3) == 3);
        load_stage(i, t + i + PF);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    for (; t < t1; t += PF) {
#pragma unroll
      for (int i = 0; i < PF; i++) {
        const int tt = t + i;
        if (tt < t1) {
          consume(i, tt, (i & 3) == 3);
          if (tt + PF < t1)
            load_stage(i, tt + PF);
        }
      }
    }
  } else {
    // one stage = G tiles; a run of 256 channels (4 tiles) closes every 4 / G stages
    auto consume_packed = [&](int i, int s) {
#pragma unroll
      for (int g = 0; g < G; g++) {
        const int tt = s * G + g;
        const i32x4 xa = *reinterpret_cast<const i32x4*>(xq_s + (tt - t0) * 16 * M + xoff);
#pragma unroll
        for (int nt = 0; nt < NTW; nt++)
          iacc[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa, sk_expand_codes<WBITS>(wreg[i][nt], g), iacc[nt], 0, 0, 0);
        if ((tt & 3) == 3) {
          const f32x4 sav = *reinterpret_cast<const f32x4*>(sa_s + ((tt >> 2) - u0) * 16 + (lane >> 4) * 4);
#pragma unroll
          for (int nt = 0; nt < NTW; nt++) {
            const float swv = sreg[i][nt] * (WBITS == 4 ? 0.0625f : 0.015625f); // operands are 16 x / 64 x the value
#pragma unroll
            for (int r = 0; r < 4; r++) {
              facc[nt][0][r] = fmaf((float)iacc[nt][r], sav[r] * swv, facc[nt][0][r]);
              iacc[nt][r] = 0;
            }
          }
        }
        if (NTW > 2)
          __builtin_amdgcn_sched_barrier(0); // one tile after the other: interleaved, the expanded operands spill
      }
    };
    const int s1 = t1 / G;
    int s = t0 / G;
    for (; s + 2 * PF <= s1; s += PF) { // branch-free full groups
#pragma unroll
      for (int i = 0; i < PF; i++) {
        consume_packed(i, s + i);
        load_stage(i, s + i + PF);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    for (; s < s1; s += PF) {
#pragma unroll
      for (int i = 0; i < PF; i++)
        if (s + i < s1) {
          consume_packed(i, s + i);
          if (s + i + PF < s1)
            load_stage(i, s + i + PF);
        }
    }
  }
  if (p.lds_overlap)
    __syncthreads(); // the reduction region overlaps the activations other waves may still be reading
  ep.finish(sg, facc, red);
}

// ---------------------------------------------------------------------------
// QINT4 / ternary QINT2 weights at their own width, 17..64 rows per block row (256-wide scale blocks): the
// activations arrive quantised in operand order (quant_act_int8_rows_kernel, as for skinny_qint8_kernel), a ring
// stage of activations is one K tile, a ring stage of weights one 16-byte load per lane and channel tile that
// holds G = 8 / WBITS consecutive K tiles (tppx_pack_qint_tiles), expanded in registers in front of the MFMA as in
// skinny_qint8_fq_kernel.  Eight waves split K in runs of 256 channels; same int32 sums, scales and fp32
// operations as skinny_qint8_kernel on the expanded tiles, so the same bits.
// ---------------------------------------------------------------------------
template <int MG, int NTW, int PF, int WBITS>
__global__ void __launch_bounds__(512)
skinny_qintx_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int G = 8 / WBITS, WS = 2, W = 8, MPAD = MG * 16;
  constexpr int UN = G * WS; // tiles per unrolled trip: 4 or 8 (a multiple of PF and of a 4-tile run)
  static_assert(UN % PF == 0 && UN % 4 == 0, "ring slots are static inside a trip");
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = blockIdx.x;
  const DecodeSeg& sg = p.seg[sk_find_seg(p, grp)];
  const int ltile0 = (grp - sg.grp0) * NTW;
  const int m0 = blockIdx.y * MPAD;
  const int NR = p.units, KT = NR * 4; // 256-wide runs (= scale blocks), K tiles
  const int u0 = (wave * NR) / W, u1 = ((wave + 1) * NR) / W;
  const int t0 = u0 * 4, t1 = u1 * 4;

  const i32x4* wq[NTW];
  const float* ws[NTW];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++) {
    const int64_t lt = min(ltile0 + nt, sg.tiles - 1); // ragged last group: duplicate, not stored
    wq[nt] = reinterpret_cast<const i32x4*>(sg.qw) + lt * (KT / G) * 64 + lane;
    ws[nt] = reinterpret_cast<const float*>(sg.sw) + lt * NR * 16 + (lane & 15);
  }
  const i32x4* xop = reinterpret_cast<const i32x4*>(p.xq) + (int64_t)blockIdx.y * MG * 64 + lane;
  const int xstride = p.mt * 64, mtp = p.mt * 16;

  i32x4 wreg[WS][NTW], xreg[PF][MG];
  float sreg[WS][NTW];
  // (past the end, or a wave without runs: re-read valid data that is never consumed -- no branch around a load)
  auto load_w = [&](int st, int gi) {
    gi = max(min(gi, t1 / G - 1), 0);
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      wreg[st][nt] = __builtin_nontemporal_load(wq[nt] + (int64_t)gi * 64);
      sreg[st][nt] = ws[nt][((gi * G) >> 2) * 16];
    }
  };
  auto load_x = [&](int st, int t) {
    t = max(min(t, t1 - 1), 0);
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      xreg[st][mg] = xop[(int64_t)t * xstride + mg * 64];
  };
#pragma unroll
  for (int i = 0; i < WS; i++)
    load_w(i, t0 / G + i);
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_x(i, t0 + i);
  __builtin_amdgcn_sched_barrier(0);
  // activation scales of this wave's runs, transposed in LDS: [u - u0][MPAD]
  float* red = sk_lds;
  float* sa_s = sk_lds + (size_t)W * NTW * MG * 256 + (size_t)wave * p.cht * MPAD;
  const int nsa = (u1 - u0) * MPAD;
  constexpr int SAB = 2 * MG;
  auto load_sa = [&](int i) {
    i = max(min(i, nsa - 1), 0);
    const int ul = i / MPAD, mr = i - ul * MPAD;
    return p.sa[(int64_t)(u0 + ul) * mtp + m0 + mr]; // [K / 256][mt * 16], written by the quantisation kernel
  };
  float sa0[SAB];
#pragma unroll
  for (int j = 0; j < SAB; j++)
    sa0[j] = load_sa(j * 64 + lane);
  __builtin_amdgcn_sched_barrier(0);
  SkEpilogue<MG, NTW, false, 8, 8> ep;
  ep.prefetch_flat(p, sg, ltile0, m0);
  __builtin_amdgcn_sched_barrier(0);
  if (t0 < t1) {
#pragma unroll
    for (int j = 0; j < SAB; j++)
      if (j * 64 + lane < nsa)
        sa_s[j * 64 + lane] = sa0[j];
    for (int i0 = SAB * 64; i0 < nsa; i0 += SAB * 64) { // more than 8 runs per wave
      float v[SAB];
#pragma unroll
      for (int j = 0; j < SAB; j++)
        v[j] = load_sa(i0 + j * 64 + lane);
#pragma unroll
      for (int j = 0; j < SAB; j++)
        if (i0 + j * 64 + lane < nsa)
          sa_s[i0 + j * 64 + lane] = v[j];
    }
  }

  f32x4 facc[NTW][MG];
  i32x4 iacc[NTW][MG];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++) {
      facc[nt][mg] = f32x4{0.f, 0.f, 0.f, 0.f};
      iacc[nt][mg] = i32x4{0, 0, 0, 0};
    }
  // tile tt: activations in stage xs, weights = part g of stage wst; a run closes every fourth tile
  auto consume = [&](int xs, int wst, int g, int tt) {
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      const i32x4 wop = sk_expand_codes<WBITS>(wreg[wst][nt], g);
#pragma unroll
      for (int mg = 0; mg < MG; mg++)
        iacc[nt][mg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xreg[xs][mg], wop, iacc[nt][mg], 0, 0, 0);
    }
    if ((tt & 3) == 3) {
#pragma unroll
      for (int mg = 0; mg < MG; mg++) {
        const f32x4 sav = *reinterpret_cast<const f32x4*>(sa_s + ((tt >> 2) - u0) * MPAD + mg * 16 + (lane >> 4) * 4);
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
          const float swv = sreg[wst][nt] * (WBITS == 4 ? 0.0625f : 0.015625f); // operands are 16 x / 64 x the value
#pragma unroll
          for (int r = 0; r < 4; r++) {
            facc[nt][mg][r] = fmaf((float)iacc[nt][mg][r], sav[r] * swv, facc[nt][mg][r]);
            iacc[nt][mg][r] = 0;
          }
        }
      }
    }
  };
  int t = t0;
  for (; t + UN <= t1; t += UN) { // branch-free full trips (reloads past the end are clamped re-reads)
#pragma unroll
    for (int i = 0; i < UN; i++) {
      consume(i % PF, (i / G) % WS, i % G, t + i);
      load_x(i % PF, t + i + PF);
      if (i % G == G - 1)
        load_w((i / G) % WS, (t + i) / G + WS);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (t < t1) { // one run left (UN == 8): its tiles are in the stages a trip would use
#pragma unroll
    for (int i = 0; i < 4; i++) {
      consume(i % PF, (i / G) % WS, i % G, t + i);
      if (i + PF < 4)
        load_x(i % PF, t + i + PF);
    }
  }
  ep.finish(sg, facc, red);
}

// ---------------------------------------------------------------------------
// W4A8 (USE_MXFP4_INT8: MXFP4 weights x int8 activations over blocks of 32, src/csrc/fused_gemm.h:965-978), M <= 16.
// The shape of skinny_qint8_fq_kernel: W waves (sixteen; eight with three channel tiles per workgroup, whose
// registers sixteen cannot hold) split K in tiles of 128 channels; a wave quantises its K
// range of the bf16 rows itself -- one (row, tile) item = 8 lanes x 16 values, the two lanes of a 32-wide block
// exchange their maxima, scale = max / 127 as quantize_int8sym, times 6 / 127 as the reference scales it -- into
// wave-private LDS in MFMA operand order, and streams the weights through a register ring.  Weight tiles are
// tppx_prepack_mxfp4_int8's: lane (channel c = lane & 15, K group kg = lane >> 4) holds four dwords, dword j = the
// eight codes of K group kg of MX block j of the tile as the reference packs them (byte i = value i | value 4 + i
// << 4), so each dword expands to the lane's operand of one K = 32 int8 MFMA = one MX block, whose exact int32 sums
// are folded into fp32 with sa[row][block] * 2^(e - 127); scales [tile][16 c] dwords of four E8M0 bytes.
// ---------------------------------------------------------------------------
template <int NTW, int PF, int XB, int W>
__global__ void __launch_bounds__(W * 64)
skinny_w4a8_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = blockIdx.x;
  const DecodeSeg& sg = p.seg[sk_find_seg(p, grp)];
  const int ltile0 = (grp - sg.grp0) * NTW;
  const int M = p.M; // <= 16
  const int KT = p.units; // K tiles of 128 channels
  const int t0 = (wave * KT) / W, t1 = ((wave + 1) * KT) / W;

  const i32x4* wq[NTW];
  const uint32_t* ws[NTW];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++) {
    const int64_t lt = min(ltile0 + nt, sg.tiles - 1);
    // (uniform bases: the lane's part stays a 32-bit offset, so the loads take scalar base + vector offset and the
    // six pointers cost no vector registers)
    wq[nt] = reinterpret_cast<const i32x4*>(sg.qw) + lt * KT * 64;
    ws[nt] = reinterpret_cast<const uint32_t*>(sg.sw) + lt * KT * 16;
  }
  // activation rows first (L2), then the post-op inputs, then the weight ring (loads return in issue order)
  const uint16_t* xb = reinterpret_cast<const uint16_t*>(p.x);
  const int nitems = M * (t1 - t0);
  const uint32_t Mu = (uint32_t)M, mmagic = p.m_magic;
  auto tile_of_item = [&](uint32_t it) { return mmagic ? __umulhi(it, mmagic) : it; }; // it / M
  i32x4 raw[XB][2];
  auto load_pass = [&](auto PS, int base) {
    constexpr int ps = decltype(PS)::value;
    const uint32_t it = (uint32_t)min((base + ps) * 8 + (lane >> 3), max(nitems - 1, 0));
    const uint32_t ul = tile_of_item(it), mr = it - ul * Mu;
    const i32x4* src = reinterpret_cast<const i32x4*>(xb + (int64_t)mr * p.K + (int64_t)(t0 + (int)ul) * 128 + (lane & 7) * 16);
    raw[ps][0] = src[0];
    raw[ps][1] = src[1];
  };
  static_for<0, XB>([&](auto PS) { load_pass(PS, 0); });
  __builtin_amdgcn_sched_barrier(0);
  SkEpilogue<1, NTW, false, W, W> ep;
  ep.prefetch_flat(p, sg, ltile0, 0);
  __builtin_amdgcn_sched_barrier(0);
  i32x4 wreg[PF][NTW];
  uint32_t sreg[PF][NTW];
  auto load_stage = [&](int st, int t) {
    t = max(min(t, t1 - 1), 0); // past the end (or a wave without tiles): re-read a valid tile, never consumed
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      wreg[st][nt] = __builtin_nontemporal_load(wq[nt] + (int64_t)t * 64 + lane);
      sreg[st][nt] = (ws[nt] + (int64_t)t * 16)[lane & 15];
    }
  };
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_stage(i, t0 + i);
  __builtin_amdgcn_sched_barrier(0);

  // wave-private LDS behind the reduction region: xq [tile][block j][K group][M rows] x 8 B, then sa [tile][j][16]
  float* red = sk_lds;
  uint8_t* mine = reinterpret_cast<uint8_t*>(sk_lds + (size_t)W * NTW * 256) + (size_t)wave * p.cht * (128 * M + 256);
  uint2* xq_s = reinterpret_cast<uint2*>(mine);
  float* sa_s = reinterpret_cast<float*>(mine + (size_t)p.cht * 128 * M);
  auto quant_pass = [&](auto PS, int base) {
    constexpr int ps = decltype(PS)::value;
    if ((base + ps) * 8 < nitems) { // wave-uniform
      const int it = (base + ps) * 8 + (lane >> 3);
      const uint32_t itc = (uint32_t)min(it, nitems - 1);
      const uint32_t ul = tile_of_item(itc), mr = itc - ul * Mu;
      float v[16];
      float amax = 0.0f;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const uint32_t wd = (uint32_t)raw[ps][j >> 2][j & 3];
        v[2 * j] = bf16_bits_to_f32(wd & 0xffffu);
        v[2 * j + 1] = bf16_bits_to_f32(wd >> 16);
        amax = fmaxf(amax, fmaxf(fabsf(v[2 * j]), fabsf(v[2 * j + 1])));
      }
      amax = sk_dpp_max<0xB1>(amax); // quad_perm [1,0,3,2]: the other half of the 32-wide block
      const float sc = __fdiv_rn(amax, 127.0f);
      const float inv = sc != 0.0f ? __frcp_rn(sc) : 0.0f;
      uint32_t pk[4];
#pragma unroll
      for (int d = 0; d < 4; d++)
        pk[d] = sk_int8x4_rne(v[4 * d], v[4 * d + 1], v[4 * d + 2], v[4 * d + 3], inv);
      if (it < nitems) {
        const int s = lane & 7, j = s >> 1, kg0 = (s & 1) * 2; // values s*16 .. of the tile: block j, K groups kg0, kg0 + 1
        uint2* dst = xq_s + (((int)ul * 4 + j) * 4 + kg0) * M + (int)mr;
        dst[0] = make_uint2(pk[0], pk[1]);
        dst[M] = make_uint2(pk[2], pk[3]);
        if ((s & 1) == 0)
          sa_s[((int)ul * 4 + j) * 16 + (int)mr] = __fmul_rn(sc, (float)(6.0 / 127.0));
      }
    }
  };
  static_for<0, XB>([&](auto PS) { quant_pass(PS, 0); });
  for (int base = XB; base * 8 < nitems; base += XB) {
    static_for<0, XB>([&](auto PS) { load_pass(PS, base); });
    static_for<0, XB>([&](auto PS) { quant_pass(PS, base); });
  }
  const int xoff = (lane >> 4) * M + min(lane & 15, M - 1); // (K group, row) inside a block's operand image

  f32x4 facc[NTW][1];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
    facc[nt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto consume = [&](int i, int tt) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint2 xa2 = xq_s[((tt - t0) * 4 + j) * 4 * M + xoff];
      const long xa = (long)(((uint64_t)xa2.y << 32) | xa2.x);
      // result rows (lane >> 4) * 4 + r; scales of rows >= M are whatever the LDS held: those rows are not stored
      const f32x4 sav = *reinterpret_cast<const f32x4*>(sa_s + ((tt - t0) * 4 + j) * 16 + (lane >> 4) * 4);
#pragma unroll
      for (int nt = 0; nt < NTW; nt++) {
        const uint32_t codes = (uint32_t)wreg[i][nt][j];
        const uint32_t lo = w4a8_expand(codes & 0x0F0F0F0Fu), hi = w4a8_expand((codes >> 4) & 0x0F0F0F0Fu);
        const long wb = (long)(((uint64_t)hi << 32) | lo);
        const i32x4 acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(xa, wb, i32x4{0, 0, 0, 0}, 0, 0, 0);
        const float wsc = e8m0_to_f32(sreg[i][nt] >> (8 * j));
#pragma unroll
        for (int r = 0; r < 4; r++)
          facc[nt][0][r] = fmaf((float)acc[r], sav[r] * wsc, facc[nt][0][r]);
      }
      if (NTW > 2)
        __builtin_amdgcn_sched_barrier(0); // one block after the other: interleaved, their temporaries spill
    }
  };
  int t = t0;
  for (; t + 2 * PF <= t1; t += PF) { // branch-free full groups: every reload is a real tile
#pragma unroll
    for (int i = 0; i < PF; i++) {
      consume(i, t + i);
      load_stage(i, t + i + PF);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (; t < t1; t += PF) {
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int tt = t + i;
      if (tt < t1) {
        consume(i, tt);
        if (tt + PF < t1)
          load_stage(i, tt + PF);
      }
    }
  }
  ep.finish(sg, facc, red);
}

// ---------------------------------------------------------------------------
// MXFP4, M <= 16, activations staged in LDS by the wave that consumes them,
// with an optional transform on the way in:
//   XMODE 0  x as it is
//   XMODE 1  RMSNorm: bf16((x * rsqrt(mean_k x^2 + eps)) * gamma[k]) -- the
//            normalisation kernel in front of the GEMM disappears
// Sixteen waves split K.  A wave reads its K slice of every row with
// row-contiguous 16-byte loads (a wave instruction covers whole 256-byte row
// segments; the operand-shaped reads of the register path touch 16 cache
// lines per 16 lanes) and writes it to its private LDS region as
// [chunk][row ^ (chunk & 15)] x 16 B: conflict free on the way in and as MFMA
// operand reads (lane = row, 4 K groups) on the way out.  The main loop then
// streams only weights.  RMSNorm needs the whole row: the 16 waves exchange
// per-(row, K tile) partial sums of squares through LDS and add them in a
// fixed order.  The reduction scratch of the epilogue reuses the x regions.
// ---------------------------------------------------------------------------
template <int NT, int PF, bool DUAL, int XMODE, int XNI>
__global__ void __launch_bounds__(1024)
skinny_mxfp4_xl_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int NTW = DUAL ? 2 * NT : NT;
  constexpr int W = 16;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = blockIdx.x;
  const int seg_id = DUAL ? 0 : sk_find_seg(p, grp);
  const DecodeSeg& sg = p.seg[seg_id];
  const int ltile0 = (grp - sg.grp0) * NT;
  const int KT = p.units;
  // K parts across workgroups (blockIdx.z of p.S, finished by finish_split): only the form that takes a K too long
  // for one workgroup's staging carries it -- a single GEMM, four channel tiles per workgroup, x as it is
  constexpr bool KSPLIT = NT == 4 && !DUAL && XMODE == 0;
  const int kt0 = KSPLIT ? ((int)blockIdx.z * KT) / p.S : 0;
  const int ktn = KSPLIT ? (((int)blockIdx.z + 1) * KT) / p.S - kt0 : KT; // K tiles of this workgroup
  const int t0 = kt0 + (wave * ktn) / W, t1 = kt0 + ((wave + 1) * ktn) / W;
  const int cht = p.cht;                       // K tiles per wave, at most
  const int wstride = max(cht * 1024, NTW * 256); // floats per wave region (x slice, later the reduction scratch)
  uint4* xs = reinterpret_cast<uint4*>(sk_lds + (size_t)wave * wstride);
  float* wss = sk_lds + (size_t)W * wstride;   // [wave][row 16][tile cht] partial sums of squares

  constexpr int NSEG = DUAL ? 2 : 1;
  const char* qwb[NSEG];
  const char* swb[NSEG];
#pragma unroll
  for (int sgi = 0; sgi < NSEG; sgi++) {
    const DecodeSeg& ss = p.seg[DUAL ? sgi : seg_id];
    qwb[sgi] = reinterpret_cast<const char*>(ss.qw);
    swb[sgi] = reinterpret_cast<const char*>(ss.sw);
  }
  uint32_t woff[NT];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
    woff[nt] = (uint32_t)(min(ltile0 + nt, sg.tiles - 1) * KT * 64 + lane);

  // ---- activations of this wave's K slice -> LDS ----
  // Loads return in issue order, so the (L2-resident) activation and gamma loads go out BEFORE the weight ring and
  // are not held up by HBM latency.  The compiler waits for exactly these ("at most the ring outstanding") as long
  // as every load between here and their first use is unconditional: a load under a branch makes its count
  // conservative, and it would wait for the ring as well, which would put everything up to the main loop behind the
  // first HBM round trip instead of inside it.
  const int nch = (t1 - t0) * 16;          // 16-byte chunks per row in the slice
  const int items = p.M * nch;             // (row, chunk), chunk fastest: 16 consecutive lanes = one K tile of one row
  const int nsh = nch > 16 ? 5 : 4;        // the host admits slices of 0, 16 or 32 chunks only
  const int cmask = (1 << nsh) - 1;
  const char* xb = reinterpret_cast<const char*>(p.x);
  const uint32_t xk0 = (uint32_t)t0 * 256u; // byte offset of the slice inside a row
  // XNI (row, chunk) items per lane: 2 cover 4 rows, 8 cover 16.  Items past the end repeat the last one (and later
  // store the same value to the same slot).  First-class vectors: the HIP struct types would stay in scratch.
  i32x4 raw[XNI];
  static_for<0, XNI>([&](auto IT) {
    constexpr int it = decltype(IT)::value;
    const int i = min(it * 64 + lane, max(items - 1, 0));
    const int row = i >> nsh, ck = i & cmask;
    const char* src = xb + (size_t)((uint32_t)(row * p.K) * 2u + xk0 + (uint32_t)ck * 16u);
    raw[it] = *reinterpret_cast<const i32x4*>(src);
  });
  // the chunk of a lane is the same in every item when the slice is 16 or 32 chunks wide
  f32x4 gm0 = f32x4{1.f, 1.f, 1.f, 1.f}, gm1 = gm0;
  if (XMODE != 0) {
    const float* gp = p.norm_gamma + (size_t)min(t0, KT - 1) * 128 + (size_t)(lane & cmask) * 8;
    gm0 = *reinterpret_cast<const f32x4*>(gp);
    gm1 = *reinterpret_cast<const f32x4*>(gp + 4);
  }
  // XMODE 2: the 256 sums of squares per row left by the launch that wrote x, 4 per lane.  Up to 4 rows (XNI == 2):
  // every wave adds up all rows itself, no exchange; more rows: wave w adds up row w and the waves exchange the
  // scales through LDS behind a barrier.
  constexpr int NPQ = XNI == 2 ? 4 : 1;
  f32x4 pq[NPQ];
  if (XMODE == 2) {
    static_for<0, NPQ>([&](auto R) {
      constexpr int r = decltype(R)::value;
      const float* sp = p.sumsq_in + (size_t)min(NPQ == 1 ? wave : r, p.M - 1) * 256 + (size_t)lane * 4;
      pq[r] = *reinterpret_cast<const f32x4*>(sp);
    });
  }

  // weight ring: it has the HBM latency to cover
  i32x4 wreg[PF][NTW];
  uint32_t sreg[PF][NTW];
  auto load_stage = [&](int st, int t) {
    t = max(min(t, t1 - 1), 0); // past the end (or a wave without K tiles): re-read a valid tile, never consumed
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      const uint32_t slot = woff[nt % NT] + (uint32_t)t * 64u;
      wreg[st][nt] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(qwb[nt / NT] + (size_t)(slot * 16u)));
      sreg[st][nt] = *reinterpret_cast<const uint8_t*>(swb[nt / NT] + (size_t)slot);
    }
  };
  // No branch around the ring's first requests and ordinary loads above: the compiler counts the ring loads behind
  // the activations itself and waits for exactly the activations (a load under a condition, or one it cannot see,
  // makes it wait for everything or not at all).
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_stage(i, t0 + i);

  // the slot arithmetic below starts from an opaque copy of the lane index, so that it is redone here instead of
  // being carried in registers across the loads above (where registers are scarcest)
  int lane2 = lane;
  asm volatile("" : "+v"(lane2));
  float* srow = wss + W * 16 * cht + wave * 16; // this wave's copy of the 16 row scales
  if (XMODE == 1) {
    // slots of rows and tiles this wave does not have count as zero
    if (lane < 16 * cht)
      wss[wave * 16 * cht + lane] = 0.f;
  }
  float rscale[NPQ]; // XMODE 2: 1/sqrt(mean square + eps) of row r (XNI == 2) or of row `wave`
  if (XMODE == 2) {
    // a row's sum in a fixed order: four entries per lane, a DPP row, the four DPP rows
    static_for<0, NPQ>([&](auto R) {
      constexpr int r = decltype(R)::value;
      float tot = (pq[r][0] + pq[r][1]) + (pq[r][2] + pq[r][3]);
      tot += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(tot), 0xB1, 0xf, 0xf, true));
      tot += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(tot), 0x4E, 0xf, 0xf, true));
      tot += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(tot), 0x141, 0xf, 0xf, true));
      tot += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(tot), 0x140, 0xf, 0xf, true));
      const float a0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tot), 0));
      const float a1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tot), 16));
      const float a2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tot), 32));
      const float a3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tot), 48));
      rscale[r] = 1.0f / sqrtf(((a0 + a1) + (a2 + a3)) * (1.0f / (float)p.K) + p.norm_eps);
    });
    if (NPQ == 1) {
      // waves past M repeat the last row into a slot nobody reads
      if (lane2 == 0)
        wss[wave] = rscale[0];
      // LDS only: a full __syncthreads would also wait for the weight ring
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
    } else {
      // through this wave's own LDS slots: selected by row in registers, the compiler turns the selection into an
      // indexed read of a stack array, a memory load that has to wait for the whole weight ring
      static_for<0, NPQ>([&](auto R) {
        if (lane2 == 0)
          srow[decltype(R)::value] = rscale[decltype(R)::value];
      });
      __builtin_amdgcn_wave_barrier();
    }
  }
  // raw activations go to their operand slots right away; the norm rescales them in place
  static_for<0, XNI>([&](auto IT) {
    constexpr int it = decltype(IT)::value;
    const int i = it * 64 + lane2;
    const int ic = min(i, max(items - 1, 0));
    const int row = ic >> nsh, ck = ic & cmask;
    if (XMODE == 1) {
      float ssq = 0.f;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t d = (uint32_t)raw[it][e];
        const float lo = bf16_bits_to_f32(d & 0xffffu), hi = bf16_bits_to_f32(d >> 16);
        ssq = fmaf(lo, lo, ssq);
        ssq = fmaf(hi, hi, ssq);
      }
      // sum over the 16 lanes of a DPP row = one (row, K tile) pair
      ssq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ssq), 0xB1, 0xf, 0xf, true));
      ssq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ssq), 0x4E, 0xf, 0xf, true));
      ssq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ssq), 0x141, 0xf, 0xf, true));
      ssq += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ssq), 0x140, 0xf, 0xf, true));
      if (i < items && (lane2 & 15) == 0)
        wss[(wave * 16 + row) * cht + (ck >> 4)] = ssq;
    }
    if (XMODE == 2) {
      // normalised on the way in: (x * scale) * gamma, one rounding
      const float sc = NPQ == 1 ? wss[row] : srow[row];
      i32x4 o;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t d = (uint32_t)raw[it][e];
        const float lo = (bf16_bits_to_f32(d & 0xffffu) * sc) * (e < 2 ? gm0[2 * e] : gm1[2 * e - 4]);
        const float hi = (bf16_bits_to_f32(d >> 16) * sc) * (e < 2 ? gm0[2 * e + 1] : gm1[2 * e - 3]);
        o[e] = (int)sk_pack_bf16(lo, hi);
      }
      *reinterpret_cast<i32x4*>(&xs[ck * 16 + (row ^ (ck & 15))]) = o;
    } else {
      *reinterpret_cast<i32x4*>(&xs[ck * 16 + (row ^ (ck & 15))]) = raw[it];
    }
  });
  if (XMODE == 1) {
    // LDS only: a full __syncthreads would also wait for the weight ring
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
    // mean of squares of whole rows in a fixed order: lane (q, r) adds waves 4q..4q+3 of row r, then the quarters
    const int q = lane >> 4, r = lane & 15;
    float tot = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < 4; w2++)
      for (int tl = 0; tl < cht; tl++)
        tot += wss[((q * 4 + w2) * 16 + r) * cht + tl];
    tot += __shfl_xor(tot, 16);
    tot += __shfl_xor(tot, 32);
    if (lane < 16)
      srow[lane] = 1.0f / sqrtf(tot * (1.0f / (float)p.K) + p.norm_eps);
    __builtin_amdgcn_wave_barrier(); // the scales are read by the other lanes of this wave
#pragma unroll 1
    for (int i = lane; i < items; i += 64) {
      const int row = i >> nsh, ck = i & cmask;
      i32x4* slot = reinterpret_cast<i32x4*>(&xs[ck * 16 + (row ^ (ck & 15))]);
      const i32x4 w = *slot;
      const float sc = srow[row];
      i32x4 o;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t d = (uint32_t)w[e];
        const float lo = (bf16_bits_to_f32(d & 0xffffu) * sc) * (e < 2 ? gm0[2 * e] : gm1[2 * e - 4]);
        const float hi = (bf16_bits_to_f32(d >> 16) * sc) * (e < 2 ? gm0[2 * e + 1] : gm1[2 * e - 3]);
        o[e] = (int)sk_pack_bf16(lo, hi);
      }
      *slot = o;
    }
  }
  // the wave reads only what it wrote itself: program order is enough

  // Nothing from below may be scheduled into the staging code above: with the normalisation's long arithmetic
  // there, the scheduler pulled the first uses of the weight ring's registers (scale conversions of the main loop)
  // up into it, and the wait for the WHOLE ring that those need landed in front of the staging (+2.4 us).
  __builtin_amdgcn_sched_barrier(0);

  // post-op inputs: requested here so that their registers are not live while the activations are in flight
  SkEpilogue<1, NTW, DUAL, 16, 16> ep;
  ep.prefetch(p, sg, ltile0, 0);

  f32x4 acc[NTW][1];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
    acc[nt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
  // operand slot of this lane for step j inside a K tile: chunk g*4 + j, row m
  int rdo[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int cj = (lane >> 4) * 4 + j;
    rdo[j] = cj * 16 + ((lane & 15) ^ cj);
  }
  auto consume = [&](int i, int tl) {
    bf16x8 xa[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
      xa[j] = __builtin_bit_cast(bf16x8, xs[tl * 256 + rdo[j]]);
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      const float sc = e8m0_to_f32(sreg[i][nt]);
#pragma unroll
      for (int j = 0; j < 4; j++)
        acc[nt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            xa[j], sk_cvt_fp4x8((uint32_t)wreg[i][nt][j], sc), acc[nt][0], 0, 0, 0);
    }
  };
  for (int t = t0; t < t1; t += PF) {
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int tt = t + i;
      if (tt < t1) {
        consume(i, tt - t0);
        if (tt + PF < t1)
          load_stage(i, tt + PF);
      }
    }
  }
  __syncthreads(); // every wave is done with its x region before it becomes reduction scratch
  if constexpr (KSPLIT) {
    if (p.S > 1) {
      ep.finish_split(p, sg, acc, sk_lds, ltile0, wstride, p.sumsq_out);
      return;
    }
  }
  ep.finish(sg, acc, sk_lds, wstride, p.sumsq_out, p.M);
}

// ---------------------------------------------------------------------------
// planning and launch
// ---------------------------------------------------------------------------
// ---------------------------------------------------------------------------
// MXFP4 weight-only, up to 4 rows, long K (the Llama down-projection of a
// batch-1 decode step): the LDS-staged kernel above with only the 4 rows kept
// -- slot (chunk, row) = chunk*4 + (row ^ (chunk & 3)); the 16 MFMA rows read
// row m & 3 -- so that K up to 16384 fits (cht KiB per wave instead of 4*cht).
// Sixteen waves split K; x and the weight ring are requested as there.
// ---------------------------------------------------------------------------
template <int NT, int PF, bool DUAL>
__global__ void __launch_bounds__(1024)
skinny_mxfp4_x4_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int NTW = DUAL ? 2 * NT : NT; // DUAL: the gate AND the up tile of each channel tile (gate tiles first)
  constexpr int W = 16, XNI = 8; // item it of a lane: row it / 2, chunk (it % 2) * 64 + lane: 4 rows x 128 chunks
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = blockIdx.x;
  const int seg_id = DUAL ? 0 : sk_find_seg(p, grp);
  const DecodeSeg& sg = p.seg[seg_id];
  const int ltile0 = (grp - sg.grp0) * NT;
  const int KT = p.units;
  const int t0 = (wave * KT) / W, t1 = ((wave + 1) * KT) / W;
  const int wstride = max(p.cht * 256, NTW * 256); // floats per wave region (x slice, later the reduction scratch)
  i32x4* xs = reinterpret_cast<i32x4*>(sk_lds + (size_t)wave * wstride);
  constexpr int NSEG = DUAL ? 2 : 1;
  const char* qwb[NSEG];
  const char* swb[NSEG];
#pragma unroll
  for (int sgi = 0; sgi < NSEG; sgi++) {
    const DecodeSeg& ss = p.seg[DUAL ? sgi : seg_id];
    qwb[sgi] = reinterpret_cast<const char*>(ss.qw);
    swb[sgi] = reinterpret_cast<const char*>(ss.sw);
  }
  uint32_t woff[NT];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
    woff[nt] = (uint32_t)(min(ltile0 + nt, sg.tiles - 1) * KT * 64 + lane);

  // activations first (L2 resident); no load below is conditional, so waiting for them does not wait for the weight ring
  const int nch = (t1 - t0) * 16;
  const char* xb = reinterpret_cast<const char*>(p.x);
  const uint32_t xk0 = (uint32_t)t0 * 256u;
  i32x4 raw[XNI];
  static_for<0, XNI>([&](auto IT) {
    constexpr int it = decltype(IT)::value;
    const int row = min(it >> 1, p.M - 1), ck = max(min((it & 1) * 64 + lane, nch - 1), 0);
    const char* src = xb + (size_t)((uint32_t)(row * p.K) * 2u + xk0 + (uint32_t)ck * 16u);
    raw[it] = *reinterpret_cast<const i32x4*>(src);
  });
  i32x4 wreg[PF][NTW];
  uint32_t sreg[PF][NTW];
  auto load_stage = [&](int st, int t) {
    t = max(min(t, t1 - 1), 0); // past the end (or a wave without K tiles): re-read a valid tile, never consumed
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      const uint32_t slot = woff[nt % NT] + (uint32_t)t * 64u;
      wreg[st][nt] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(qwb[nt / NT] + (size_t)(slot * 16u)));
      sreg[st][nt] = *reinterpret_cast<const uint8_t*>(swb[nt / NT] + (size_t)slot);
    }
  };
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_stage(i, t0 + i); // no branch around these: the compiler then counts them and waits for the activations only
  int lane2 = lane;
  asm volatile("" : "+v"(lane2));
  static_for<0, XNI>([&](auto IT) {
    constexpr int it = decltype(IT)::value;
    const i32x4 v = raw[it];
    const int row = it >> 1, ck = (it & 1) * 64 + lane2;
    if (row < p.M && ck < nch)
      xs[ck * 4 + (row ^ (ck & 3))] = v;
  });
  // the wave reads only what it wrote itself: program order is enough

  SkEpilogue<1, NTW, DUAL, 16, 16> ep;
  ep.prefetch(p, sg, ltile0, 0);
  f32x4 acc[NTW][1];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
    acc[nt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
  // operand slot of this lane for step j inside a K tile: chunk g*4 + j (+ 16 per tile), row m & 3
  int rdo[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int cj = (lane >> 4) * 4 + j;
    rdo[j] = cj * 4 + ((lane & 3) ^ (cj & 3));
  }
  auto consume = [&](int i, int tl) {
    bf16x8 xa[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
      xa[j] = __builtin_bit_cast(bf16x8, xs[tl * 64 + rdo[j]]);
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      const float sc = e8m0_to_f32(sreg[i][nt]);
#pragma unroll
      for (int j = 0; j < 4; j++)
        acc[nt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            xa[j], sk_cvt_fp4x8((uint32_t)wreg[i][nt][j], sc), acc[nt][0], 0, 0, 0);
    }
  };
  int t = t0;
  for (; t + 2 * PF <= t1; t += PF) { // branch-free full groups: every reload is a real tile
#pragma unroll
    for (int i = 0; i < PF; i++) {
      consume(i, t + i - t0);
      load_stage(i, t + i + PF);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (; t < t1; t += PF) {
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int tt = t + i;
      if (tt < t1) {
        consume(i, tt - t0);
        if (tt + PF < t1)
          load_stage(i, tt + PF);
      }
    }
  }
  __syncthreads(); // every wave is done with its x region before it becomes reduction scratch
  ep.finish(sg, acc, sk_lds, wstride, p.sumsq_out, p.M);
}

// ---------------------------------------------------------------------------
// MXFP4 weight-only, 17..64 rows: MG row groups of 16 per workgroup.
// Eight waves split K.  A wave walks its K tiles one at a time: the bf16
// activations of the tile (MG*16 rows x 256 B, row-contiguous 16-byte loads,
// requested a tile ahead into registers) are written to the wave's private
// LDS region in MFMA operand order -- slot (chunk, row) = chunk*MPAD + (row ^
// chunk), the same conflict-free image the 16-row kernel uses -- and read back
// as A operands; every dequantised weight operand feeds MG MFMAs.  No barrier
// before the final cross-wave reduction, no operand-shaped global loads, no
// second kernel.  The epilogue's reduction scratch reuses the activation
// regions.
// ---------------------------------------------------------------------------
template <int MG, int NT, bool DUAL, int PF, int W = 8, bool XLATE = false>
__global__ void __launch_bounds__(W * 64)
skinny_mxfp4_mg_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int MPAD = MG * 16, XL = MG * 4;
  constexpr int NTW = DUAL ? 2 * NT : NT; // DUAL: the gate AND the up tile of each channel tile (gate tiles first)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = blockIdx.x;
  const int seg_id = DUAL ? 0 : sk_find_seg(p, grp);
  const DecodeSeg& sg = p.seg[seg_id];
  const int ltile0 = (grp - sg.grp0) * NT;
  const int m0 = blockIdx.y * MPAD;
  const int KT = p.units;
  // K tiles of this workgroup (all of them unless K is split across workgroups), then of this wave
  const int tb = sk_share(blockIdx.z, KT, p.S), te = sk_share(blockIdx.z + 1, KT, p.S);
  const int t0 = tb + (wave * (te - tb)) / W, t1 = tb + ((wave + 1) * (te - tb)) / W;
  i32x4* xs = reinterpret_cast<i32x4*>(sk_lds) + (size_t)wave * (MPAD * 16); // [chunk 16][row MPAD] x 16 B

  constexpr int NSEG = DUAL ? 2 : 1;
  const char* qwb[NSEG];
  const char* swb[NSEG];
#pragma unroll
  for (int sgi = 0; sgi < NSEG; sgi++) {
    const DecodeSeg& ss = p.seg[DUAL ? sgi : seg_id];
    qwb[sgi] = reinterpret_cast<const char*>(ss.qw);
    swb[sgi] = reinterpret_cast<const char*>(ss.sw);
  }
  uint32_t woff[NT];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
    woff[nt] = (uint32_t)(min(ltile0 + nt, sg.tiles - 1) * KT * 64 + lane);

  // activation item `it` of this lane: row it*4 + lane/16 of the block row, chunk lane%16 of the tile's 256 bytes;
  // rows past M re-read row M-1 (their results are not stored)
  const char* xb = reinterpret_cast<const char*>(p.x);
  const int r4 = lane >> 4, c16 = lane & 15;
  // The per-item addresses are cheap to derive and expensive to keep (2 * XL registers): both helpers start from
  // opaque copies of the lane coordinates so that the compiler rebuilds them at every call instead of hoisting them
  // out of the K loop.
  i32x4 xr[XL];
  auto load_x = [&](int t) {
    t = max(min(t, t1 - 1), 0); // past the end (or a wave without K tiles): a valid tile, never consumed
    int r = r4, c = c16;
    asm volatile("" : "+v"(r), "+v"(c));
    const uint32_t base = (uint32_t)t * 256u + (uint32_t)c * 16u;
#pragma unroll
    for (int it = 0; it < XL; it++) {
      const int row = min(m0 + it * 4 + r, p.M - 1);
      xr[it] = *reinterpret_cast<const i32x4*>(xb + (size_t)((uint32_t)(row * p.K) * 2u + base));
    }
  };
  auto store_x = [&]() {
    int r = r4, c = c16;
    asm volatile("" : "+v"(r), "+v"(c));
#pragma unroll
    for (int it = 0; it < XL; it++)
      xs[c * MPAD + ((it * 4 + r) ^ c)] = xr[it];
  };
  // operand slot of this lane for step j: chunk g*4 + j, row m of row group mg (+ mg*16)
  int rdo[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int cj = (lane >> 4) * 4 + j;
    rdo[j] = cj * MPAD + ((lane & 15) ^ cj);
  }

  i32x4 wreg[PF][NTW];
  uint32_t sreg[PF][NTW];
  auto load_stage = [&](int st, int t) {
    t = max(min(t, t1 - 1), 0); // past the end (or a wave without K tiles): a valid tile, never consumed
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      const uint32_t slot = woff[nt % NT] + (uint32_t)t * 64u;
      wreg[st][nt] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(qwb[nt / NT] + (size_t)(slot * 16u)));
      sreg[st][nt] = *reinterpret_cast<const uint8_t*>(swb[nt / NT] + (size_t)slot);
    }
  };
  // (no branch around the first requests: the compiler then counts the ring behind the activations and waits for
  // the activations only)
  load_x(t0); // needed first, requested first
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_stage(i, t0 + i);
  // post-op inputs early, except where registers are scarcest (the gate/up pair has none but its biases)
  constexpr bool LATE_EP = DUAL && MG == 4;
  SkEpilogue<MG, NTW, DUAL, W, W> ep;
  if (!LATE_EP)
    ep.prefetch(p, sg, ltile0, m0);

  f32x4 acc[NTW][MG];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      acc[nt][mg] = f32x4{0.f, 0.f, 0.f, 0.f};

  // one K tile: activations of the tile into LDS, the next tile's requested, then 4 steps x MG x NT MFMAs
  // XLATE (the widest variants, 96 accumulators): the next tile's activations are requested BEHIND the tile's MFMAs,
  // where the 64 staging registers are free, instead of in front of them -- that makes room for a second stage of
  // the weight ring (with one stage the next tile's weights can only be requested after the tile's last MFMA and are
  // needed right away).  Measured level with the one-stage form (64-row gate/up pair 24.4 against 24.6 us): a wave
  // waits a memory round trip per K tile either way, for its weights there and for its activations here; both
  // prefetches together need 188 bytes of scratch per lane.
  auto consume = [&](int i, int tnext) {
    store_x();
    if (!XLATE)
      load_x(tnext);
    float sc[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++)
      sc[nt] = e8m0_to_f32(sreg[i][nt]);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      // NT dequantised operands at a time (DUAL: the gate tiles, then the up tiles; the activation operands are
      // read again, which is cheaper than keeping either set in registers)
#pragma unroll
      for (int h = 0; h < NTW / NT; h++) {
        bf16x8 b[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
          b[nt] = sk_cvt_fp4x8((uint32_t)wreg[i][h * NT + nt][j], sc[h * NT + nt]);
#pragma unroll
        for (int mg = 0; mg < MG; mg++) {
          const bf16x8 a = __builtin_bit_cast(bf16x8, xs[rdo[j] + mg * 16]);
#pragma unroll
          for (int nt = 0; nt < NT; nt++)
            acc[h * NT + nt][mg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[nt], acc[h * NT + nt][mg], 0, 0, 0);
        }
        if (MG * NT >= 12)
          __builtin_amdgcn_sched_barrier(0); // widest variants: keep the operands of one group live at a time
      }
    }
  };
  int t = t0;
  for (; t + 2 * PF <= t1; t += PF) { // branch-free full groups: every reload is a real tile, wait counts stay exact
#pragma unroll
    for (int i = 0; i < PF; i++) {
      consume(i, t + i + 1);
      if (XLATE) {
        __builtin_amdgcn_sched_barrier(0);
        load_x(t + i + 1); // in front of the weights: loads return in issue order
      }
      load_stage(i, t + i + PF);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (; t < t1; t += PF) {
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int tt = t + i;
      if (tt < t1) {
        consume(i, tt + 1);
        if (XLATE) {
          __builtin_amdgcn_sched_barrier(0);
          load_x(tt + 1);
        }
        if (tt + PF < t1)
          load_stage(i, tt + PF);
      }
    }
  }
  if (LATE_EP)
    ep.prefetch(p, sg, ltile0, m0);
  __syncthreads(); // every wave is done with its activation region before it becomes reduction scratch
  if constexpr (DUAL) {
    ep.finish_halves(sg, acc, sk_lds);
  } else {
    if (p.S > 1)
      ep.finish_split(p, sg, acc, sk_lds, ltile0);
    else
      ep.finish(sg, acc, sk_lds, decltype(ep)::ELEMS, p.sumsq_out, p.M);
  }
}

// ---------------------------------------------------------------------------
// Unquantized bf16 weights (the reference's default lm_head), any number of
// rows: the row-group kernel above without the dequantisation.  Native tiles
// hold the MFMA operands themselves, [N/16][K/128][4 j][64 lanes][16 B], so a
// K tile of a channel tile is four 1 KB loads per wave; activations go
// through the same wave-private LDS image.  Block rows of MG*16 rows ride on
// grid y: beyond 64 rows every block row streams the weights again (from L2
// / Infinity Cache when they fit), which is what a prompt's last-token
// lm_head or a short verification batch needs, not a prefill GEMM.
// ---------------------------------------------------------------------------
template <int MG, int NT, int PF, int W>
__global__ void __launch_bounds__(W * 64)
skinny_bf16_kernel(const DecodeParams p) {
  extern __shared__ __align__(16) float sk_lds[];
  constexpr int MPAD = MG * 16, XL = MG * 4;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = blockIdx.x;
  const DecodeSeg& sg = p.seg[sk_find_seg(p, grp)];
  const int ltile0 = (grp - sg.grp0) * NT;
  const int m0 = blockIdx.y * MPAD;
  const int KT = p.units;
  const int t0 = (wave * KT) / W, t1 = ((wave + 1) * KT) / W;
  i32x4* xs = reinterpret_cast<i32x4*>(sk_lds) + (size_t)wave * (MPAD * 16); // [chunk 16][row MPAD] x 16 B

  const i32x4* wb = reinterpret_cast<const i32x4*>(sg.qw);
  size_t woff[NT]; // in 16-byte units
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
    woff[nt] = (size_t)min(ltile0 + nt, sg.tiles - 1) * KT * 256 + lane;

  const char* xb = reinterpret_cast<const char*>(p.x);
  const int r4 = lane >> 4, c16 = lane & 15;
  i32x4 xr[XL];
  auto load_x = [&](int t) {
    t = max(min(t, t1 - 1), 0); // past the end (or a wave without K tiles): a valid tile, never consumed
    int r = r4, c = c16;
    asm volatile("" : "+v"(r), "+v"(c));
    const size_t base = (size_t)t * 256u + (size_t)c * 16u;
#pragma unroll
    for (int it = 0; it < XL; it++) {
      const int row = min(m0 + it * 4 + r, p.M - 1);
      xr[it] = *reinterpret_cast<const i32x4*>(xb + (size_t)row * p.K * 2u + base);
    }
  };
  auto store_x = [&]() {
    int r = r4, c = c16;
    asm volatile("" : "+v"(r), "+v"(c));
#pragma unroll
    for (int it = 0; it < XL; it++)
      xs[c * MPAD + ((it * 4 + r) ^ c)] = xr[it];
  };
  int rdo[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int cj = (lane >> 4) * 4 + j;
    rdo[j] = cj * MPAD + ((lane & 15) ^ cj);
  }

  i32x4 wreg[PF][NT][4];
  auto load_stage = [&](int st, int t) {
    t = max(min(t, t1 - 1), 0); // past the end (or a wave without K tiles): a valid tile, never consumed
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        wreg[st][nt][j] = __builtin_nontemporal_load(wb + woff[nt] + (size_t)t * 256 + j * 64);
  };
  load_x(t0); // no branch around the first requests (exact wait counts)
#pragma unroll
  for (int i = 0; i < PF; i++)
    load_stage(i, t0 + i);
  SkEpilogue<MG, NT, false, W, W> ep;
  ep.prefetch(p, sg, ltile0, m0);

  f32x4 acc[NT][MG];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
#pragma unroll
    for (int mg = 0; mg < MG; mg++)
      acc[nt][mg] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto consume = [&](int i, int tnext) {
    store_x();
    load_x(tnext);
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int mg = 0; mg < MG; mg++) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, xs[rdo[j] + mg * 16]);
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
          acc[nt][mg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, wreg[i][nt][j]), acc[nt][mg], 0, 0, 0);
      }
  };
  int t = t0;
  for (; t + 2 * PF <= t1; t += PF) { // branch-free full groups: every reload is a real tile
#pragma unroll
    for (int i = 0; i < PF; i++) {
      consume(i, t + i + 1);
      load_stage(i, t + i + PF);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (; t < t1; t += PF) {
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int tt = t + i;
      if (tt < t1) {
        consume(i, tt + 1);
        if (tt + PF < t1)
          load_stage(i, tt + PF);
      }
    }
  }
  __syncthreads(); // every wave is done with its activation region before it becomes reduction scratch
  ep.finish(sg, acc, sk_lds, decltype(ep)::ELEMS);
}

// Scale blocks that `runs` consecutive runs of `deal` tiles can touch (slots of activation scales a wave keeps in LDS).
int skinny_qint8_blocks_per_wave(int runs, int tpb, int deal, int nblk) {
  const int tiles = runs * deal;
  int n = (deal % tpb == 0) ? tiles / tpb : (tiles + tpb - 1) / tpb + 1; // whole blocks : a range that starts anywhere
  if (n > nblk)
    n = nblk;
  return n < 1 ? 1 : n;
}

// launch shape of the QINT8 decode kernels
SkinnyPlan plan_skinny(int64_t M, int total_tiles, int units, int tpb, int deal, bool can_fuse_quant) {
  const int env_ntw = env_int("TPPX_SKINNY_NTW", 0), env_waves = env_int("TPPX_SKINNY_WAVES", 0),
            env_fusedq = env_int("TPPX_SKINNY_FUSEDQ", 1);
  SkinnyPlan pl;
  const int nblk = (int)((int64_t)units * deal / tpb);
  const int mrows = (int)(M < 64 ? M : 64);
  pl.mg = mrows <= 16 ? 1 : (mrows <= 32 ? 2 : 4);
  pl.grid_y = (int)((M + 16 * pl.mg - 1) / (16 * pl.mg));
  // two channel tiles per wave once there are plenty of tiles: halves the
  // activation-operand traffic per weight byte
  pl.ntw = total_tiles >= 512 ? 2 : 1;
  if (env_ntw == 1 || env_ntw == 2)
    pl.ntw = env_ntw;
  // more than 16 rows: these kernels run one workgroup per CU, so prefer a grid
  // of at most 256 workgroups (a second, partly filled round costs a full one)
  if (pl.mg > 1 && env_ntw == 0 && total_tiles > 512 && total_tiles <= 768)
    pl.ntw = 3;
  // Wave-count window of the kernel instantiation that will run (register
  // budget: 16 waves leave 128 VGPRs per lane, 8 leave 256; the epilogue's
  // outputs-per-thread bound sets the minimum).  Waves beyond the number of
  // runs of K simply get an empty range.
  const bool wide = pl.mg == 4 || (pl.mg == 2 && pl.ntw >= 2);
  const int max_w = wide ? 8 : 16, min_w = wide ? 8 : 4;
  // few tiles: one 16-wave workgroup per CU keeps the whole weight in flight
  int w = env_waves > 0 ? env_waves : ((total_tiles / pl.ntw <= 320) ? 16 : 8);
  if (w > units)
    w = units;
  if (w > max_w)
    w = max_w;
  if (w < min_w)
    w = min_w;
  pl.waves = w;
  pl.max_units = skinny_qint8_blocks_per_wave((units + w - 1) / w, tpb, deal, nblk);
  pl.fused_quant = false;
  pl.lds_overlap = false;
  if (M <= 16 && can_fuse_quant && env_fusedq != 0) {
    // quantisation inside the GEMM kernel: 16 waves, the fewest channel tiles per workgroup that keep the grid
    // within one round of 256 workgroups, as long as the quantised rows of all waves fit the LDS
    const int ntw = total_tiles <= 256 ? 1 : (total_tiles <= 512 ? 2 : 3);
    const int cht = (units + 15) / 16; // runs of 256 input channels per wave
    const bool bigb = tpb > 4;         // blocks of several runs: maxima exchanged between the waves, items in registers
    const size_t abytes = bigb ? (size_t)M * units * sizeof(float) : 0;
    const size_t xbytes = (size_t)16 * cht * (256 * (size_t)M + 64) + abytes, rbytes = (size_t)16 * ntw * 1024;
    const int xb = bigb ? (ntw == 1 ? 6 : 4) : 0;
    if (xbytes <= 160 * 1024 && rbytes <= 160 * 1024 && (!bigb || M * (int64_t)cht <= 4 * xb)) {
      pl.fused_quant = true;
      pl.lds_overlap = xbytes + rbytes > 160 * 1024;
      pl.ntw = ntw;
      pl.waves = 16;
      pl.max_units = cht;
    }
  }
  return pl;
}

int skinny_split_tickets(int n) {
  static std::mutex mu;
  static int cursor = 0;
  if (n <= 0 || n > SK_TICKETS)
    return -1;
  std::lock_guard<std::mutex> lock(mu);
  if (cursor + n > SK_TICKETS)
    cursor = 0;
  const int first = cursor;
  cursor += n;
  return first;
}

// A launch that the runtime refused leaves its counter window as it found it, but whoever gets the window next
// relies on zeros: clear it on the way out (a fill kernel, so the call may sit inside a stream capture).
__global__ void sk_clear_tickets_kernel(int first, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    sk_split_tickets[first + i] = 0;
}

template <typename K>
static hipError_t sk_launch(K kern, const DecodeParams& p, dim3 grid, int waves, size_t lds, hipStream_t stream) {
  TPPX_PLAN_ONLY(kern, grid, dim3(64 * waves), lds);
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
  if (e == hipSuccess) {
    kern<<<grid, dim3(64 * waves), lds, stream>>>(p);
    e = hipGetLastError();
  }
  if (e != hipSuccess && grid.z > 1 && p.ticket0 >= 0) {
    const int n = (int)(grid.x * grid.y);
    sk_clear_tickets_kernel<<<dim3((n + 255) / 256), dim3(256), 0, stream>>>(p.ticket0, n);
    (void)hipGetLastError(); // the caller reports the launch's own error
  }
  return e;
}

// groups are counted per segment by the caller with the same ntw
hipError_t launch_skinny_qint8(DecodeParams& p, const SkinnyPlan& pl, hipStream_t stream) {
  p.cht = pl.max_units; // per-wave slots of activation scales in LDS
  dim3 grid(p.groups, pl.grid_y, pl.fused_quant ? 1 : p.S);
  if (grid.z > 1 && (p.S > 4 || (p.ticket0 = skinny_split_tickets((int)(grid.x * grid.y))) < 0))
    return hipErrorInvalidValue;
  p.tpb_magic = p.tpb > 1 ? (unsigned int)(((1ull << 32) + (unsigned int)p.tpb - 1) / (unsigned int)p.tpb) : 0u;
  if (pl.fused_quant) {
    p.m_magic = p.M > 1 ? (unsigned int)(((1ull << 32) + (unsigned int)p.M - 1) / (unsigned int)p.M) : 0u;
    const bool bigb = p.tpb > 4;
    const size_t abytes = bigb ? (size_t)p.M * p.units * sizeof(float) : 0;
    const size_t xbytes = (size_t)16 * pl.max_units * (256 * (size_t)p.M + 64) + abytes, rbytes = (size_t)16 * pl.ntw * 1024;
    const size_t lds = pl.lds_overlap ? (xbytes > rbytes ? xbytes : rbytes) : xbytes + rbytes;
    p.lds_overlap = pl.lds_overlap ? 1 : 0;
    if (p.wbits == 4 || p.wbits == 2) { // packed codes (256-wide blocks; the caller checks)
#define SKQX(NTW, XB)                                                                                           \
  return p.wbits == 4 ? sk_launch(skinny_qint8_fq_kernel<NTW, 4, 16, 16, XB, false, 4>, p, grid, 16, lds, stream) \
                      : sk_launch(skinny_qint8_fq_kernel<NTW, (NTW == 3 ? 2 : 4), 16, 16, XB, false, 2>, p, grid, 16, lds, stream)
      if (pl.ntw == 3)
        SKQX(3, 2);
      if (pl.ntw == 2)
        SKQX(2, 4);
      if ((int64_t)p.M * pl.max_units > 16)
        SKQX(1, 6);
      SKQX(1, 4);
#undef SKQX
    }
    if (bigb) { // all (row, run) items of a wave stay in registers: M * runs per wave <= 4 * XB (plan_skinny checked)
      if (pl.ntw == 3)
        return sk_launch(skinny_qint8_fq_kernel<3, 4, 16, 16, 4, true>, p, grid, 16, lds, stream);
      if (pl.ntw == 2)
        return sk_launch(skinny_qint8_fq_kernel<2, 4, 16, 16, 4, true>, p, grid, 16, lds, stream);
      if (pl.max_units <= 3) // (the ring of eight is slower here too: 16.8 against 15.6 us at 8 rows x 11008)
        return sk_launch(skinny_qint8_fq_kernel<1, 4, 16, 16, 6, true>, p, grid, 16, lds, stream);
      return sk_launch(skinny_qint8_fq_kernel<1, 8, 16, 16, 6, true>, p, grid, 16, lds, stream);
    }
    if (pl.ntw == 3)
      return sk_launch(skinny_qint8_fq_kernel<3, 4, 16, 16, 2, false>, p, grid, 16, lds, stream);
    if (pl.ntw == 2)
      return sk_launch(skinny_qint8_fq_kernel<2, 4, 16, 16, 4, false>, p, grid, 16, lds, stream);
    // Up to three K blocks (12 weight tiles) per wave: a ring of four tiles; one of eight would hold most of the
    // wave's K range and only delays its first MFMA (4096 x 4096 at one row 6.9 -> 5.9 us).  With more than 16
    // (row, block) items per wave, six quantisation passes are in flight, so that up to 24 items (8 rows x 3 blocks
    // of the K = 11008 down-projection) are requested before the weight ring and none queues behind it
    // (14.0 -> 12.2 us).  From four blocks per wave on the ring of eight wins.
    if (pl.max_units <= 3) {
      if ((int64_t)p.M * pl.max_units > 16)
        return sk_launch(skinny_qint8_fq_kernel<1, 4, 16, 16, 6, false>, p, grid, 16, lds, stream);
      return sk_launch(skinny_qint8_fq_kernel<1, 4, 16, 16, 4, false>, p, grid, 16, lds, stream);
    }
    return sk_launch(skinny_qint8_fq_kernel<1, 8, 16, 16, 4, false>, p, grid, 16, lds, stream);
  }
  size_t lds = ((size_t)pl.waves * pl.ntw * pl.mg * 256 + (size_t)pl.waves * pl.max_units * pl.mg * 16) * sizeof(float);
#define SKQ(MG, NTW, PF, MAXW, MINW)                                                                   \
  return p.mt > 0 ? sk_launch(skinny_qint8_kernel<MG, NTW, PF, MAXW, MINW, true>, p, grid, pl.waves, lds, stream) \
                  : sk_launch(skinny_qint8_kernel<MG, NTW, PF, MAXW, MINW, false>, p, grid, pl.waves, lds, stream)
  if (pl.ntw == 3) {
    if (pl.mg == 2)
      SKQ(2, 3, 4, 8, 8);
    SKQ(4, 3, 2, 8, 8); // (225 registers; a ring of three or four stages spills 620 / 164 bytes per lane)
  }
  if (pl.ntw == 2) {
    switch (pl.mg) {
      case 1: SKQ(1, 2, 4, 16, 4);
      case 2: SKQ(2, 2, 8, 8, 8);
      default: SKQ(4, 2, 4, 8, 8);
    }
  }
  switch (pl.mg) {
    case 1: SKQ(1, 1, 4, 16, 4);
    case 2: SKQ(2, 1, 4, 16, 4);
    default:
      // a ring of four: one of eight spills 36 bytes per lane, and scratch costs far more than the deeper ring gains
      // (4096 x 4096 at 64 rows: 11.9 us with it, 9.8 us without)
      if (p.mt > 0)
        return sk_launch(skinny_qint8_kernel<4, 1, 4, 8, 8, true>, p, grid, pl.waves, lds, stream);
      return sk_launch(skinny_qint8_kernel<4, 1, 4, 8, 8, false>, p, grid, pl.waves, lds, stream);
  }
#undef SKQ
}

// 17..32 (mg = 2) or 33..64 (mg = 4) rows per block row, four channel tiles x four K parts per workgroup, K in p.S slices across workgroups
// (grid x = channel groups * S); p.units = 256-wide runs of K, activations in operand order (p.mt > 0)
template <int MG, int TW, int KPW, int WPF, int XPF, int MAXSTEPS>
static hipError_t sk_launch_nk(const DecodeParams& p, dim3 grid, hipStream_t stream) {
  const size_t stage = ((size_t)2 * KPW * 4 * MG * 256 + 2 * KPW * 64) * sizeof(float);
  const size_t redb = (size_t)KPW * TW * MG * 256 * sizeof(float);
  const size_t lds = stage > redb ? stage : redb;
  const auto kern = skinny_qint8_nk_kernel<MG, TW, KPW, WPF, XPF, MAXSTEPS>;
  TPPX_PLAN_ONLY(kern, grid, dim3(TW * KPW * 64), lds);
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
  if (e == hipSuccess) {
    kern<<<grid, dim3(TW * KPW * 64), lds, stream>>>(p);
    e = hipGetLastError();
  }
  return e;
}

hipError_t launch_skinny_qint8_nk(DecodeParams& p, int mg, hipStream_t stream) {
  const int groups = (p.total_tiles + 3) / 4, grid_y = (p.M + mg * 16 - 1) / (mg * 16);
  dim3 grid(groups * p.S, grid_y, 1);
  if (p.S > 4 || p.n_seg != 1 || p.mt <= 0 || p.deal != 4)
    return hipErrorInvalidValue;
  if (p.S > 1 && (p.ticket0 = skinny_split_tickets(groups * grid_y)) < 0)
    return hipErrorInvalidValue;
  // steps of a wave: runs of a K slice over the four K parts
  const int nsteps = ((p.units + p.S - 1) / p.S + 3) / 4;
  if (nsteps > 8)
    return hipErrorInvalidValue;
  // weights three steps ahead, activations one: deeper rings spill at 128 registers (+4 us), two and two is level
  hipError_t e = mg == 2 ? sk_launch_nk<2, 4, 4, 3, 1, 8>(p, grid, stream) : sk_launch_nk<4, 4, 4, 3, 1, 8>(p, grid, stream);
  if (e != hipSuccess && p.S > 1 && p.ticket0 >= 0 && !plan_recording()) {
    const int n = groups * grid_y;
    sk_clear_tickets_kernel<<<dim3((n + 255) / 256), dim3(256), 0, stream>>>(p.ticket0, n);
    (void)hipGetLastError();
  }
  return e;
}

// QINT4 / QINT2 codes at their own width, 17..64 rows per block row (p.wbits, p.mt set; 256-wide blocks, one K part)
hipError_t launch_skinny_qintx(DecodeParams& p, int mg, int ntw, hipStream_t stream) {
  if ((p.wbits != 4 && p.wbits != 2) || p.S != 1 || p.mt <= 0 || p.deal != 4 || p.tpb != 4 || (mg != 2 && mg != 4) ||
      ntw < 1 || ntw > 3)
    return hipErrorInvalidValue;
  p.cht = (p.units + 7) / 8; // runs of a wave: slots of activation scales in LDS
  dim3 grid(p.groups, (p.M + mg * 16 - 1) / (mg * 16), 1);
  const size_t lds = ((size_t)8 * ntw * mg * 256 + (size_t)8 * p.cht * mg * 16) * sizeof(float);
  // activations two tiles ahead at four row groups, four at two (the register budget of eight waves per workgroup)
#define SKQR(MG, NTW)                                                                                            \
  if (mg == MG && ntw == NTW)                                                                                    \
    return p.wbits == 4 ? sk_launch(skinny_qintx_kernel<MG, NTW, (MG == 4 ? 2 : 4), 4>, p, grid, 8, lds, stream) \
                        : sk_launch(skinny_qintx_kernel<MG, NTW, (MG == 4 ? 2 : 4), 2>, p, grid, 8, lds, stream);
  SKQR(2, 1) SKQR(2, 2) SKQR(2, 3) SKQR(4, 1) SKQR(4, 2) SKQR(4, 3)
#undef SKQR
  return hipErrorInvalidValue;
}

// W4A8, M <= 16, weights prepacked by tppx_prepack_mxfp4_int8; false when the quantised rows do not fit the LDS
bool skinny_w4a8_fits(int64_t M, int total_tiles, int ktiles, int* ntw_out) {
  const int ntw = total_tiles <= 256 ? 1 : (total_tiles <= 512 ? 2 : 3);
  const int w = ntw == 3 ? 8 : 16;
  const int cht = (ktiles + w - 1) / w;
  const size_t xbytes = (size_t)w * cht * (128 * (size_t)M + 256), rbytes = (size_t)w * ntw * 1024;
  *ntw_out = ntw;
  return M >= 1 && M <= 16 && xbytes + rbytes <= 160 * 1024;
}

hipError_t launch_skinny_w4a8(DecodeParams& p, int ntw, hipStream_t stream) {
  const int w = ntw == 3 ? 8 : 16;
  p.cht = (p.units + w - 1) / w;
  p.m_magic = p.M > 1 ? (unsigned int)(((1ull << 32) + (unsigned int)p.M - 1) / (unsigned int)p.M) : 0u;
  dim3 grid(p.groups, 1, 1);
  const size_t lds = (size_t)w * p.cht * (128 * (size_t)p.M + 256) + (size_t)w * ntw * 1024;
  // a wave holds at most four K tiles at the 7B shapes: a ring of four (two with two channel tiles: registers)
  switch (ntw) {
    case 1: return sk_launch(skinny_w4a8_kernel<1, 4, 4, 16>, p, grid, 16, lds, stream);
    case 2: return sk_launch(skinny_w4a8_kernel<2, 2, 4, 16>, p, grid, 16, lds, stream);
    default: return sk_launch(skinny_w4a8_kernel<3, 4, 4, 8>, p, grid, 8, lds, stream);
  }
}

// MXFP4, 33..64 rows per block row: four channel tiles x four K parts per workgroup, K in p.S slices across workgroups
hipError_t launch_skinny_mxfp4_nk(DecodeParams& p, hipStream_t stream) {
  const int groups = (p.total_tiles + 3) / 4, grid_y = (p.M + 63) / 64;
  dim3 grid(groups * p.S, grid_y, 1);
  const int nsteps = ((p.units + p.S - 1) / p.S + 3) / 4;
  if (p.S > 4 || p.n_seg != 1 || nsteps > 8)
    return hipErrorInvalidValue;
  if (p.S > 1 && (p.ticket0 = skinny_split_tickets(groups * grid_y)) < 0)
    return hipErrorInvalidValue;
  const size_t lds = (size_t)2 * 4 * 64 * 16 * 16; // two stages x four K parts x 64 rows x 256 B (> the reduction's 64 KiB)
  const int form = env_int("TPPX_MXFP4_NK_FORM", 0);
  hipError_t e;
  if (form == 1) { // one tile per wave, sixteen waves
    const auto kern = skinny_mxfp4_nk_kernel<4, 4, 1, 4, 6, 2, 8>;
    TPPX_PLAN_ONLY(kern, grid, dim3(1024), lds);
    e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
    if (e == hipSuccess) {
      kern<<<grid, dim3(1024), lds, stream>>>(p);
      e = hipGetLastError();
    }
  } else { // two tiles per wave, eight waves: half the operand reads from LDS per MFMA
    const auto kern = skinny_mxfp4_nk_kernel<4, 4, 2, 4, 6, 2, 8>;
    TPPX_PLAN_ONLY(kern, grid, dim3(512), lds);
    e = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds);
    if (e == hipSuccess) {
      kern<<<grid, dim3(512), lds, stream>>>(p);
      e = hipGetLastError();
    }
  }
  if (e != hipSuccess && p.S > 1 && p.ticket0 >= 0) {
    const int n = groups * grid_y;
    sk_clear_tickets_kernel<<<dim3((n + 255) / 256), dim3(256), 0, stream>>>(p.ticket0, n);
    (void)hipGetLastError();
  }
  return e;
}

// x staged in LDS, optional fused RMSNorm; 16 waves; nt = channel tiles per workgroup (of each GEMM when dual)
size_t skinny_mxfp4_xl_lds(int units, int nt, bool dual) {
  const int cht = (units + 15) / 16;
  const int ntw = dual ? 2 * nt : nt;
  const size_t wstride = (size_t)(cht * 1024 > ntw * 256 ? cht * 1024 : ntw * 256);
  return (16 * wstride + (size_t)16 * 16 * cht + 16 * 16) * sizeof(float);
}

hipError_t launch_skinny_mxfp4_xl(DecodeParams& p, int nt, bool dual, hipStream_t stream) {
  // p.S > 1 (nt == 4, single GEMM, no normalisation; the caller checks): K parts across workgroups, every part staged
  // like a whole K of its length
  const int S = p.S > 1 ? p.S : 1;
  const int units = (p.units + S - 1) / S;
  p.cht = (units + 15) / 16;
  const size_t lds = skinny_mxfp4_xl_lds(units, nt, dual);
  dim3 grid(p.groups, 1, S);
  if (S > 1 && (S > 4 || nt != 4 || dual || p.norm_gamma || (p.ticket0 = skinny_split_tickets((int)grid.x)) < 0))
    return hipErrorInvalidValue;
  const bool norm = p.norm_gamma != nullptr;
  const bool few = p.M <= 4; // 4 rows x 32 chunks fit two items per lane
  const bool handed = norm && p.sumsq_in != nullptr; // row sums of squares come from the launch that wrote x
#define SKXL(NT, DUAL)                                                                                       \
  return handed ? (few ? sk_launch(skinny_mxfp4_xl_kernel<NT, 2, DUAL, 2, 2>, p, grid, 16, lds, stream)      \
                       : sk_launch(skinny_mxfp4_xl_kernel<NT, 2, DUAL, 2, 8>, p, grid, 16, lds, stream))     \
       : norm   ? (few ? sk_launch(skinny_mxfp4_xl_kernel<NT, 2, DUAL, 1, 2>, p, grid, 16, lds, stream)      \
                       : sk_launch(skinny_mxfp4_xl_kernel<NT, 2, DUAL, 1, 8>, p, grid, 16, lds, stream))     \
                : (few ? sk_launch(skinny_mxfp4_xl_kernel<NT, 2, DUAL, 0, 2>, p, grid, 16, lds, stream)      \
                       : sk_launch(skinny_mxfp4_xl_kernel<NT, 2, DUAL, 0, 8>, p, grid, 16, lds, stream))
  if (dual) {
    if (nt == 3)
      SKXL(3, true);
    if (nt == 2)
      SKXL(2, true);
    SKXL(1, true);
  }
  if (nt == 4)
    SKXL(4, false);
  if (nt == 3)
    SKXL(3, false);
  if (nt == 2)
    SKXL(2, false);
  SKXL(1, false);
#undef SKXL
}

// up to 4 rows, K up to 16384 (8 tiles per wave); nt = channel tiles per workgroup (1..3; of each GEMM when dual)
hipError_t launch_skinny_mxfp4_x4(DecodeParams& p, int nt, bool dual, hipStream_t stream) {
  p.cht = (p.units + 15) / 16;
  const int ntw = dual ? 2 * nt : nt;
  const size_t wstride = (size_t)(p.cht * 256 > ntw * 256 ? p.cht * 256 : ntw * 256);
  const size_t lds = 16 * wstride * sizeof(float);
  dim3 grid(p.groups, 1);
  if (dual) {
    if (nt == 3)
      return sk_launch(skinny_mxfp4_x4_kernel<3, 2, true>, p, grid, 16, lds, stream);
    if (nt == 2)
      return sk_launch(skinny_mxfp4_x4_kernel<2, 2, true>, p, grid, 16, lds, stream);
    return sk_launch(skinny_mxfp4_x4_kernel<1, 4, true>, p, grid, 16, lds, stream);
  }
  if (nt == 3)
    return sk_launch(skinny_mxfp4_x4_kernel<3, 2, false>, p, grid, 16, lds, stream);
  if (nt == 2)
    return sk_launch(skinny_mxfp4_x4_kernel<2, 4, false>, p, grid, 16, lds, stream);
  return sk_launch(skinny_mxfp4_x4_kernel<1, 4, false>, p, grid, 16, lds, stream);
}

size_t skinny_mxfp4_mg_lds(int mg, int ntw, int waves) {
  const size_t xbytes = (size_t)waves * mg * 16 * 256, rbytes = (size_t)waves * ntw * mg * 1024;
  return xbytes > rbytes ? xbytes : rbytes;
}

// mg = 1, 2 or 4 row groups of 16 per block row; nt = channel tiles per workgroup (1..4; of each GEMM when dual);
// groups counted by the caller
hipError_t launch_skinny_mxfp4_mg(DecodeParams& p, int mg, int nt, bool dual, hipStream_t stream) {
  dim3 grid(p.groups, (p.M + mg * 16 - 1) / (mg * 16), p.S);
  if (p.S > 1 && (p.S > 4 || (p.ticket0 = skinny_split_tickets((int)(grid.x * grid.y))) < 0))
    return hipErrorInvalidValue;
  if (mg == 1) { // up to 16 rows: sixteen waves, deeper weight ring
    const size_t lds1 = skinny_mxfp4_mg_lds(1, nt, 16);
#define SKMG1(NT, DUAL, PF) return sk_launch(skinny_mxfp4_mg_kernel<1, NT, DUAL, PF, 16>, p, grid, 16, lds1, stream)
    if (dual) {
      if (nt == 3)
        SKMG1(3, true, 1);
      if (nt == 2)
        SKMG1(2, true, 2);
      SKMG1(1, true, 4);
    }
    if (nt == 3)
      SKMG1(3, false, 4);
    if (nt == 2)
      SKMG1(2, false, 4);
    SKMG1(1, false, 4);
#undef SKMG1
  }
  const size_t lds = skinny_mxfp4_mg_lds(mg, nt, 8); // the gate/up pair is reduced one half at a time
#define SKMG(MG, NT, DUAL, PF) return sk_launch(skinny_mxfp4_mg_kernel<MG, NT, DUAL, PF>, p, grid, 8, lds, stream)
#define SKMGL(MG, NT, DUAL, PF) return sk_launch(skinny_mxfp4_mg_kernel<MG, NT, DUAL, PF, 8, true>, p, grid, 8, lds, stream)
  if (dual) {
    if (mg == 2) {
      if (nt == 3)
        SKMG(2, 3, true, 2);
      if (nt == 2)
        SKMG(2, 2, true, 2);
      SKMG(2, 1, true, 2);
    }
    if (nt == 3) {
      if (env_int("TPPX_MXFP4_MG_LATE", 1) != 0)
        SKMGL(4, 3, true, 2); // 96 accumulators: two ring stages with the activations requested behind the MFMAs
      SKMG(4, 3, true, 1);    // ... or one stage with them requested in front (64 staging registers live)
    }
    if (nt == 2)
      SKMG(4, 2, true, 2);
    SKMG(4, 1, true, 2);
  }
  if (mg == 2) {
    if (nt == 4)
      SKMG(2, 4, false, 2);
    if (nt == 3)
      SKMG(2, 3, false, 2);
    if (nt == 2)
      SKMG(2, 2, false, 2);
    SKMG(2, 1, false, 2);
  }
  if (nt == 4) {
    if (env_int("TPPX_MXFP4_MG_LATE", 1) != 0)
      SKMGL(4, 4, false, 2);
    SKMG(4, 4, false, 1);
  }
  if (nt == 3)
    SKMG(4, 3, false, 2);
  if (nt == 2)
    SKMG(4, 2, false, 2);
  SKMG(4, 1, false, 2);
#undef SKMG
#undef SKMGL
}

// bf16 weights: mg row groups of 16 per block row (1, 2 or 4), nt channel tiles per workgroup (1 or 2)
hipError_t launch_skinny_bf16(DecodeParams& p, int mg, int nt, hipStream_t stream) {
  dim3 grid(p.groups, (p.M + mg * 16 - 1) / (mg * 16), 1);
  if (mg == 1) {
    const size_t lds1 = skinny_mxfp4_mg_lds(1, nt, 16);
    if (nt == 2)
      return sk_launch(skinny_bf16_kernel<1, 2, 2, 16>, p, grid, 16, lds1, stream);
    return sk_launch(skinny_bf16_kernel<1, 1, 4, 16>, p, grid, 16, lds1, stream);
  }
  const size_t lds = skinny_mxfp4_mg_lds(mg, nt, 8);
#define SKBF(MG, NT, PF) return sk_launch(skinny_bf16_kernel<MG, NT, PF, 8>, p, grid, 8, lds, stream)
  if (mg == 2) {
    if (nt == 2)
      SKBF(2, 2, 2);
    SKBF(2, 1, 2);
  }
  if (nt == 2)
    SKBF(4, 2, 2);
  SKBF(4, 1, 2);
#undef SKBF
}

} // namespace tppx
