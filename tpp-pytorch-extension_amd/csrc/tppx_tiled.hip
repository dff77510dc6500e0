// Prefill-shape (large M) LDS-tiled MFMA kernels.
//
// Workgroup tile 128 (M) x 128 (N), 4 waves in a 2 x 2 grid, each wave 64 x 64
// = 4 x 4 MFMA tiles of 16 x 16.  Per K step of 128 input channels:
//   A (activations): global -> registers -> LDS, stored in MFMA operand order
//     so that a wave-wide ds_read_b128 is lane-contiguous (conflict free); two
//     LDS buffers, the global loads of step k+1 are in flight while step k is
//     multiplied.
//   B (weights): the native 1 KiB tiles ARE the MFMA operand layout, so every
//     wave loads its four channel tiles straight from global/L2 into registers
//     (one 128-bit load per lane and tile, next step prefetched) - no LDS, no
//     re-layout.  MXFP4 codes are expanded to bf16 in registers with the
//     hardware E8M0-scaled convert (exact) and multiplied with
//     v_mfma_f32_16x16x32_bf16; QINT8 uses v_mfma_i32_16x16x64_i8 with exact
//     int32 sums per K block and an fp32 scale-and-accumulate.
// Workgroup ids are remapped so that the workgroups of one XCD (ids equal
// mod 8) walk consecutive M blocks of the same N block: the weight tiles of
// that N block stay in the XCD's L2.
//
// MFMA operand convention (A = activations, B = weights):
//   lane l supplies row/col (l & 15) and K group (l >> 4);
//   result register r of lane l is D[m = (l >> 4) * 4 + r][n = l & 15].
#include <algorithm>
#include <string.h>
#include <type_traits>

#include "tppx_common.h"
#include "tppx_launch.h"

namespace tppx {

__device__ __forceinline__ bf16x8 tl_cvt_fp4x8(uint32_t codes, float scale) {
  bf16x2 c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 0);
  bf16x2 c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 1);
  bf16x2 c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 2);
  bf16x2 c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 3);
  bf16x8 w;
  w[0] = c0[0]; w[1] = c0[1]; w[2] = c1[0]; w[3] = c1[1];
  w[4] = c2[0]; w[5] = c2[1]; w[6] = c3[0]; w[7] = c3[1];
  return w;
}

// XCD-aware tile order: returns (bm, bn) of this workgroup.  Workgroup ids go round the 8 XCDs; XCD x gets a
// rectangle of the tile space and walks it row block fastest, so that the workgroups resident on an XCD at the same
// time share operand tiles in its L2.  xm = how many of the 8 rectangles lie along M (1: an XCD owns NB/8 channel
// blocks and all row blocks; 2, 4: 1/xm of the row blocks and xm/8 of the channel blocks).  Every XCD fetches
// 1/xm of the activations and xm/8 of the weights from memory.  The host passes an xm that divides evenly.
__device__ __forceinline__ void tile_of_block(int MB, int NB, int& bm, int& bn, int xm = 1) {
  int id = blockIdx.x;
  const int T = MB * NB;
  if ((T & 7) == 0 && xm > 1) {
    const int x = id & 7, r = id >> 3;
    const int xn = 8 / xm;                // rectangles along N
    const int mb = MB / xm, nb = NB / xn; // the rectangle of XCD x: mb x nb tiles at (x % xm, x / xm)
    bm = (x % xm) * mb + r % mb;
    bn = (x / xm) * nb + r / mb;
    return;
  }
  if ((T & 7) == 0) { // an eighth of the tiles in column-major order, whether or not NB divides by 8
    const int per = T >> 3;
    id = (id & 7) * per + (id >> 3);
  }
  bm = id % MB;
  bn = id / MB;
}

template <typename Acc>
__device__ __forceinline__ void tiled_epilogue(const TiledParams& p, Acc& acc, int m_base, int tile_base) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int tile = tile_base + nt;
    if (tile >= p.tiles)
      continue;
    const int n = tile * 16 + (lane & 15);
    const float b = p.bias ? bf16_bits_to_f32(p.bias[n]) : 0.0f;
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int m = m_base + mt * 16 + (lane >> 4) * 4 + r;
        if (m < p.M) {
          const int64_t o = (int64_t)m * p.N + n;
          uint32_t in1 = p.post_in ? p.post_in[o] : 0u;
          uint32_t in2 = p.post_in2 ? p.post_in2[o] : 0u;
          p.y[o] = (uint16_t)apply_post_bits(acc[mt][nt][r] + b, p.post_op, in1, in2, p.post_scale);
        }
      }
  }
}

// ---------------------------------------------------------------------------
// MXFP4, bf16 activations (exact reference numerics, fp32 accumulation over K)
// LDS A layout per buffer: [mt 8][j 4][lane 64] x 16 B  (32 KiB)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
tiled_mxfp4_kernel(const TiledParams p) {
  extern __shared__ __align__(16) uint8_t tl_lds[];
  bf16x8* As = reinterpret_cast<bf16x8*>(tl_lds); // 2 buffers x 2048 slots
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int MB = (p.M + 127) >> 7, NB = (p.tiles + 7) >> 3;
  int bm, bn;
  tile_of_block(MB, NB, bm, bn);
  const int KT = p.K >> 7; // K steps of 128 = native tiles along K
  const int m_wg = bm * 128;
  const int tile_base = bn * 8 + wn * 4;

  const i32x4* wq[4];
  const uint8_t* wsc[4];
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int64_t t = min(tile_base + nt, p.tiles - 1);
    wq[nt] = reinterpret_cast<const i32x4*>(p.qw) + t * KT * 64 + lane;
    wsc[nt] = reinterpret_cast<const uint8_t*>(p.sw) + t * KT * 64 + lane;
  }
  // A staging: thread handles LDS slots tid + 256*q  ->  (r16, g, j = wave, mt = q)
  const uint16_t* xb = reinterpret_cast<const uint16_t*>(p.x);
  const uint16_t* arow[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    const int m = min(m_wg + q * 16 + (tid & 15), p.M - 1);
    arow[q] = xb + (int64_t)m * p.K + ((tid >> 4) & 3) * 32 + wave * 8;
  }

  bf16x8 areg[8];
  i32x4 breg[4];
  uint32_t bsc[4];
  auto load_a = [&](int ks) {
#pragma unroll
    for (int q = 0; q < 8; q++)
      areg[q] = *reinterpret_cast<const bf16x8*>(arow[q] + ks * 128);
  };
  auto load_b = [&](int ks) {
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      breg[nt] = wq[nt][(int64_t)ks * 64];
      bsc[nt] = wsc[nt][(int64_t)ks * 64];
    }
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 8; q++)
      As[buf * 2048 + q * 256 + tid] = areg[q];
  };

  f32x4 acc[4][4];
#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  load_a(0);
  load_b(0);
  store_a(0);
  __syncthreads();
  for (int ks = 0; ks < KT; ks++) {
    const int buf = ks & 1;
    i32x4 bcur[4];
    float sc[4];
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      bcur[nt] = breg[nt];
      sc[nt] = e8m0_to_f32(bsc[nt]);
    }
    if (ks + 1 < KT) {
      load_a(ks + 1);
      load_b(ks + 1);
    }
    const bf16x8* Ab = As + buf * 2048 + (wm * 4) * 256 + lane;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      bf16x8 a[4], b[4];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
        a[mt] = Ab[mt * 256 + j * 64];
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        b[nt] = tl_cvt_fp4x8((uint32_t)bcur[nt][j], sc[nt]);
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[mt], b[nt], acc[mt][nt], 0, 0, 0);
    }
    if (ks + 1 < KT)
      store_a(buf ^ 1);
    __syncthreads();
  }
  tiled_epilogue(p, acc, m_wg + wm * 64, tile_base);
}

// ---------------------------------------------------------------------------
// Unquantized bf16 weights at prefill shapes (the prompt pass of a model whose
// first-token weights stay bf16): the kernel above without the expansion.  The
// native bf16 tiles [N/16][K/128][4 j][64 lanes][16 B] hold the MFMA operands
// themselves, 4 KiB per (channel tile, K step) -- eight times the bytes of the
// packed codes -- so B runs as a ring of the four steps j of a K step: the
// operand of (ks, j) is requested right behind the MFMAs that consumed
// (ks - 1, j), a whole K step ahead, and no second register set is needed.
// All loads are ordinary register loads, so the compiler's partial waits hold.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
tiled_bf16_kernel(const TiledParams p) {
  extern __shared__ __align__(16) uint8_t tl_lds[];
  bf16x8* As = reinterpret_cast<bf16x8*>(tl_lds); // 2 buffers x 2048 slots
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int MB = (p.M + 127) >> 7, NB = (p.tiles + 7) >> 3;
  int bm, bn;
  tile_of_block(MB, NB, bm, bn);
  const int KT = p.K >> 7;
  const int m_wg = bm * 128;
  const int tile_base = bn * 8 + wn * 4;

  const i32x4* wq[4];
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int64_t t = min(tile_base + nt, p.tiles - 1);
    wq[nt] = reinterpret_cast<const i32x4*>(p.qw) + t * KT * 256 + lane;
  }
  const uint16_t* xb = reinterpret_cast<const uint16_t*>(p.x);
  const uint16_t* arow[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    const int m = min(m_wg + q * 16 + (tid & 15), p.M - 1);
    arow[q] = xb + (int64_t)m * p.K + ((tid >> 4) & 3) * 32 + wave * 8;
  }
  bf16x8 areg[8];
  i32x4 bring[4][4]; // [j][nt]
  auto load_a = [&](int ks) {
#pragma unroll
    for (int q = 0; q < 8; q++)
      areg[q] = *reinterpret_cast<const bf16x8*>(arow[q] + ks * 128);
  };
  auto load_b = [&](int ks, int j) {
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      bring[j][nt] = wq[nt][(int64_t)ks * 256 + j * 64];
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 8; q++)
      As[buf * 2048 + q * 256 + tid] = areg[q];
  };

  f32x4 acc[4][4];
#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  load_a(0);
#pragma unroll
  for (int j = 0; j < 4; j++)
    load_b(0, j);
  store_a(0);
  __syncthreads();
  for (int ks = 0; ks < KT; ks++) {
    const int buf = ks & 1;
    const bool more = ks + 1 < KT;
    if (more)
      load_a(ks + 1);
    const bf16x8* Ab = As + buf * 2048 + (wm * 4) * 256 + lane;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      bf16x8 a[4];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
        a[mt] = Ab[mt * 256 + j * 64];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[mt], __builtin_bit_cast(bf16x8, bring[j][nt]), acc[mt][nt], 0, 0, 0);
      if (more)
        load_b(ks + 1, j);
    }
    if (more)
      store_a(buf ^ 1);
    __syncthreads();
  }
  tiled_epilogue(p, acc, m_wg + wm * 64, tile_base);
}

// ---------------------------------------------------------------------------
// QINT8 (W8A8): activations pre-quantised (int8 [M][K], f32 [M][K/qbs]).
// K step = 128 = two native tiles; LDS A layout per buffer:
// [mt 8][t 2][lane 64] x 16 B (16 KiB) + the activation scales of the step's
// K block for the 128 rows.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256, 2) // two workgroups per CU: without the bound the compiler spreads into 327 registers, one wave per SIMD
tiled_qint8_kernel(const TiledParams p) {
  extern __shared__ __align__(16) uint8_t tl_lds[];
  i32x4* As = reinterpret_cast<i32x4*>(tl_lds);                 // 2 x 1024 slots
  float* sa_s = reinterpret_cast<float*>(tl_lds + 2 * 1024 * 16); // 2 x 128
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int MB = (p.M + 127) >> 7, NB = (p.tiles + 7) >> 3;
  int bm, bn;
  tile_of_block(MB, NB, bm, bn);
  const int KS = p.K >> 7;        // K steps of 128
  const int KT = p.K >> 6;        // native tiles along K
  const int SPB = p.qbs >> 7;     // steps per K block (qbs is a multiple of 128 here)
  const int NBK = p.K / p.qbs;
  const int m_wg = bm * 128;
  const int tile_base = bn * 8 + wn * 4;

  const i32x4* wq[4];
  const float* wsc[4];
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int64_t t = min(tile_base + nt, p.tiles - 1);
    wq[nt] = reinterpret_cast<const i32x4*>(p.qw) + t * KT * 64 + lane;
    wsc[nt] = reinterpret_cast<const float*>(p.sw) + t * NBK * 16 + (lane & 15);
  }
  // A staging: slots tid + 256*q -> (r16, g, t = wave & 1, mt = 2*q + (wave >> 1))
  const int8_t* xq = reinterpret_cast<const int8_t*>(p.xq);
  const int8_t* arow[4];
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int mt = q * 2 + (wave >> 1);
    const int m = min(m_wg + mt * 16 + (tid & 15), p.M - 1);
    arow[q] = xq + (int64_t)m * p.K + (wave & 1) * 64 + ((tid >> 4) & 3) * 16;
  }
  const int sa_row = min(m_wg + (tid & 127), p.M - 1);

  i32x4 areg[4], breg[2][4];
  float sareg = 0.f;
  auto load_a = [&](int ks) {
#pragma unroll
    for (int q = 0; q < 4; q++)
      areg[q] = *reinterpret_cast<const i32x4*>(arow[q] + ks * 128);
    if (ks % SPB == 0 && tid < 128)
      sareg = p.sa[(int64_t)sa_row * NBK + ks / SPB];
  };
  auto load_b = [&](int ks) {
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        breg[t][nt] = wq[nt][(int64_t)(ks * 2 + t) * 64];
  };
  auto store_a = [&](int ks, int buf) {
#pragma unroll
    for (int q = 0; q < 4; q++)
      As[buf * 1024 + q * 256 + tid] = areg[q];
    if (ks % SPB == 0 && tid < 128)
      sa_s[((ks / SPB) & 1) * 128 + tid] = sareg;
  };

  f32x4 facc[4][4];
  i32x4 iacc[4][4];
#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      facc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
      iacc[mt][nt] = i32x4{0, 0, 0, 0};
    }

  load_a(0);
  load_b(0);
  store_a(0, 0);
  __syncthreads();
  for (int ks = 0; ks < KS; ks++) {
    const int buf = ks & 1;
    i32x4 bcur[2][4];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        bcur[t][nt] = breg[t][nt];
    if (ks + 1 < KS) {
      load_a(ks + 1);
      load_b(ks + 1);
    }
    // slot = (mt*2 + t)*64 + lane with mt = wm*4 + i
    const i32x4* Ab = As + buf * 1024 + (wm * 4) * 128 + lane;
#pragma unroll
    for (int t = 0; t < 2; t++) {
      i32x4 a[4];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
        a[mt] = Ab[mt * 128 + t * 64];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
          iacc[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[mt], bcur[t][nt], iacc[mt][nt], 0, 0, 0);
    }
    if ((ks + 1) % SPB == 0) { // K block complete: scale and fold into fp32
      const int b = ks / SPB;
      const float* sab = sa_s + (b & 1) * 128 + wm * 64 + (lane >> 4) * 4;
      float swv[4];
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        swv[nt] = wsc[nt][b * 16];
#pragma unroll
      for (int mt = 0; mt < 4; mt++) {
        const f32x4 sav = *reinterpret_cast<const f32x4*>(sab + mt * 16);
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            facc[mt][nt][r] = fmaf((float)iacc[mt][nt][r], sav[r] * swv[nt], facc[mt][nt][r]);
            iacc[mt][nt][r] = 0;
          }
      }
    }
    if (ks + 1 < KS)
      store_a(ks + 1, buf ^ 1);
    __syncthreads();
  }
  tiled_epilogue(p, facc, m_wg + wm * 64, tile_base);
}

// ---------------------------------------------------------------------------
// Large-M MXFP4 kernel: workgroup tile 256 (M) x 256 (N), 8 waves in a 2 x 4
// grid (two per SIMD), each wave 128 x 64 = 8 x 4 MFMA tiles (128 accumulator
// registers).  Every expanded weight operand feeds 8 MFMAs, every activation
// operand read from LDS feeds 4 and is requested two MFMA groups ahead.
//   A: 4 rows x 256 B per wave instruction go from global memory straight
//      into LDS (global_load_lds, no staging registers), a whole K step ahead,
//      two buffers of 64 KiB.  The LDS image of such a load is lane-linear, so
//      the bank swizzle is applied on the source side: the lane at position c
//      of row m fetches chunk c ^ (m & 15), and the operand reads of a K group
//      fall on 16 different bank groups.
//   B: native tiles straight from global/L2, fetched half a K step ahead.
// LDS byte address of chunk ck of row m of row tile mt:
//   mt*4096 + (m>>2)*1024 + (m&3)*256 + ((ck ^ m) & 15)*16.
// ---------------------------------------------------------------------------
// Epilogue of a 128 x 64 wave tile through a wave-private LDS region: the
// fp32 sums of 64 rows at a time are written there (statically indexed, so the
// accumulators stay in registers), then read back row-contiguously; every
// lane finishes 8 adjacent channels and writes them with one 16-byte store.
constexpr int EP_LD = 68; // floats per staged row: 64 + 4 keeps the 4-row lane groups on distinct banks
template <int MT>
__device__ __forceinline__ void big_epilogue(const TiledParams& p, f32x4 (&acc)[MT][4], float* stage, int m_base,
                                             int tile_base) {
  const int lane = threadIdx.x & 63;
  const int cx = (lane & 7) * 8; // first of this lane's 8 channels inside the wave tile
  const int tile = tile_base + (cx >> 4);
  const bool tile_ok = tile < p.tiles;
  const int n = min(tile, p.tiles - 1) * 16 + (cx & 15);
  float bias[8];
#pragma unroll
  for (int e = 0; e < 8; e++)
    bias[e] = p.bias ? bf16_bits_to_f32(p.bias[n + e]) : 0.0f;
  constexpr int MH = MT < 4 ? MT : 4; // row tiles staged at a time (64 rows, or the whole wave tile when it has fewer)
#pragma unroll
  for (int h = 0; h < MT / MH; h++) {
#pragma unroll
    for (int mt = 0; mt < MH; mt++)
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          stage[(mt * 16 + (lane >> 4) * 4 + r) * EP_LD + nt * 16 + (lane & 15)] = acc[h * MH + mt][nt][r];
    // same wave wrote and reads: no barrier, the compiler orders the LDS accesses
    for (int it = 0; it < MH * 2; it++) {
      const int row = it * 8 + (lane >> 3);
      const int m = m_base + h * (MH * 16) + row;
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(stage + row * EP_LD + cx);
      const f32x4 v1 = *reinterpret_cast<const f32x4*>(stage + row * EP_LD + cx + 4);
      if (tile_ok && m < p.M) {
        const int64_t o = (int64_t)m * p.N + n;
        uint4 i1 = make_uint4(0, 0, 0, 0), i2 = make_uint4(0, 0, 0, 0);
        if (p.post_in)
          i1 = *reinterpret_cast<const uint4*>(p.post_in + o);
        if (p.post_in2)
          i2 = *reinterpret_cast<const uint4*>(p.post_in2 + o);
        const uint32_t w1[4] = {i1.x, i1.y, i1.z, i1.w}, w2[4] = {i2.x, i2.y, i2.z, i2.w};
        uint32_t out[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float lo = (e < 2 ? v0[2 * e] : v1[2 * e - 4]) + bias[2 * e];
          const float hi = (e < 2 ? v0[2 * e + 1] : v1[2 * e - 3]) + bias[2 * e + 1];
          const uint32_t a = apply_post_bits(lo, p.post_op, w1[e] & 0xffffu, w2[e] & 0xffffu, p.post_scale);
          const uint32_t b = apply_post_bits(hi, p.post_op, w1[e] >> 16, w2[e] >> 16, p.post_scale);
          out[e] = (a & 0xffffu) | (b << 16);
        }
        *reinterpret_cast<uint4*>(p.y + o) = make_uint4(out[0], out[1], out[2], out[3]);
      }
    }
  }
}

// The gate/up pair: the wave tile's channels 0..31 are gate sums and 32..63 the up sums of the SAME 32 output
// channels, so silu(gate) * up is formed here, with the rounding points of SiluPostOp followed by MulPostOp, and
// only the product is written: a lane finishes 8 adjacent channels of one row (16-byte store, four lanes per row).
template <int MT>
__device__ __forceinline__ void big_epilogue_dual(const TiledParams& pg, const TiledParams& pu, f32x4 (&acc)[MT][4],
                                                  float* stage, int m_base, int tile_base) {
  const int lane = threadIdx.x & 63;
  const int cx = (lane & 3) * 8; // first of this lane's 8 channels among the wave's 32
  const int tile = tile_base + (cx >> 4);
  const bool tile_ok = tile < pg.tiles;
  const int n = min(tile, pg.tiles - 1) * 16 + (cx & 15);
  float bg[8], bu[8];
#pragma unroll
  for (int e = 0; e < 8; e++) {
    bg[e] = pg.bias ? bf16_bits_to_f32(pg.bias[n + e]) : 0.0f;
    bu[e] = pu.bias ? bf16_bits_to_f32(pu.bias[n + e]) : 0.0f;
  }
  constexpr int MH = MT < 4 ? MT : 4; // row tiles staged at a time
#pragma unroll
  for (int h = 0; h < MT / MH; h++) {
#pragma unroll
    for (int mt = 0; mt < MH; mt++)
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          stage[(mt * 16 + (lane >> 4) * 4 + r) * EP_LD + nt * 16 + (lane & 15)] = acc[h * MH + mt][nt][r];
    // same wave wrote and reads: no barrier, the compiler orders the LDS accesses
    for (int it = 0; it < MH; it++) {
      const int row = it * 16 + (lane >> 2);
      const int m = m_base + h * (MH * 16) + row;
      const f32x4 g0 = *reinterpret_cast<const f32x4*>(stage + row * EP_LD + cx);
      const f32x4 g1 = *reinterpret_cast<const f32x4*>(stage + row * EP_LD + cx + 4);
      const f32x4 u0 = *reinterpret_cast<const f32x4*>(stage + row * EP_LD + 32 + cx);
      const f32x4 u1 = *reinterpret_cast<const f32x4*>(stage + row * EP_LD + 32 + cx + 4);
      if (tile_ok && m < pg.M) {
        uint32_t out[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float glo = (e < 2 ? g0[2 * e] : g1[2 * e - 4]) + bg[2 * e];
          const float ghi = (e < 2 ? g0[2 * e + 1] : g1[2 * e - 3]) + bg[2 * e + 1];
          const float ulo = (e < 2 ? u0[2 * e] : u1[2 * e - 4]) + bu[2 * e];
          const float uhi = (e < 2 ? u0[2 * e + 1] : u1[2 * e - 3]) + bu[2 * e + 1];
          const uint32_t ga = apply_post_bits(glo, TPPX_POST_SILU, 0, 0, 1.0f);
          const uint32_t gb = apply_post_bits(ghi, TPPX_POST_SILU, 0, 0, 1.0f);
          const uint32_t a = apply_post_bits(ulo, TPPX_POST_MUL, ga & 0xffffu, 0, 1.0f);
          const uint32_t b = apply_post_bits(uhi, TPPX_POST_MUL, gb & 0xffffu, 0, 1.0f);
          out[e] = (a & 0xffffu) | (b << 16);
        }
        *reinterpret_cast<uint4*>(pu.y + (int64_t)m * pu.N + n) = make_uint4(out[0], out[1], out[2], out[3]);
      }
    }
  }
}

// LDS operand reads issued by hand, so that they can be kept several MFMA
// groups ahead of their use: the compiler does not track them, the waits are
// explicit (LDS operations complete in issue order, so "at most N younger
// operations outstanding" is enough) and are tied to the destination
// registers so that nothing using them can move above the wait.
template <int OFF>
__device__ __forceinline__ void lds_read_b128_async(i32x4& dst, uint32_t byte_addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(byte_addr), "n"(OFF));
}
template <int N>
__device__ __forceinline__ void lds_wait_keep(i32x4& r) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "n"(N));
}

// Several GEMMs over one activation (fused q/k/v) share a launch: the channel
// blocks of all segments form one grid.
struct BigParams {
  TiledParams seg[TPPX_MAX_SEGS];
  int nb0[TPPX_MAX_SEGS + 1]; // first channel block of each segment, then the total
  int n_seg;
  int xm;                     // XCD rectangles along M (see tile_of_block)
};

// MT = 16-row tiles per wave along M (8).
// DUAL: the gate/up pair (seg[0] = gate, seg[1] = up, equal shapes).  A workgroup owns 128 output channels and
// computes their gate AND up sums (wave tile = 2 gate tiles + the 2 up tiles of the same channels); the epilogue
// writes silu(gate) * up once.  Channel blocks are 128 wide then.
// WM x WN waves, each with a wave tile of MT*16 rows x 64 channels:
//   2 x 4  workgroup tile 256 x 256, one workgroup per CU
//   1 x 4  128 x 256, 4 waves, TWO workgroups per CU: half-size workgroups for shapes whose last round of 256-row
//          workgroups would be mostly empty
//   1 x 8  128 x 512, one workgroup per CU: the same 65536 sums per CU as 2 x 4, but half the activation bytes per
//          K step (128 rows) and every weight tile fetched by ONE wave instead of by the two of a wave column -- half
//          the bytes moved from L2 into the CU per MFMA
// WBF16: unquantized bf16 weights in their native tiles ([N/16][K/128][4 j][64 lanes][16 B], the MFMA operands
// themselves) instead of packed codes + scales: 16 bytes per lane, tile and MFMA step, so they run as a ring of the
// four steps j of a K step -- (ks + 1, j) is requested right behind the last MFMA group of (ks, j), a whole K step
// ahead -- and no second register set is needed.  These loads are issued and waited for by hand (they complete in
// issue order, so "at most N younger loads outstanding" is the wait): with loads into LDS pending the compiler
// answers the first use of any loaded register, and the fence of __syncthreads(), with a wait for ALL loads.
template <int MT, bool DUAL, int WM, int WN, bool WBF16>
__device__ __forceinline__ void big_gemm_body(const BigParams& P) {
  static_assert(!WBF16 || !DUAL, "the bf16-weight form: single GEMMs");
  constexpr int WGM = MT * 16 * WM; // rows per workgroup
  constexpr int NBLK = MT * 4 / WN; // blocks of 4 rows x 256 B of the A tile that a wave fetches per K step
  static_assert(NBLK % 4 == 0, "the swizzle below takes a wave's first block to be a multiple of 4");
  constexpr int ABUF = WGM * 256;  // bytes of one A buffer (rows x 128 K bf16)
  extern __shared__ __align__(16) uint8_t tl_lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform: keeps LDS bases and block indices scalar
  const int wm = wave % WM, wn = wave / WM;
  const int MB = (P.seg[0].M + WGM - 1) / WGM;
  int bm, bn;
  tile_of_block(MB, P.nb0[P.n_seg], bm, bn, P.xm);
  // pick this block's GEMM with uniform selects (everything stays in scalar registers)
  TiledParams p = P.seg[0];
  int nb_first = 0;
  if (!DUAL) {
#pragma unroll
    for (int i = 1; i < TPPX_MAX_SEGS; i++)
      if (i < P.n_seg && bn >= P.nb0[i]) {
        p = P.seg[i];
        nb_first = P.nb0[i];
      }
  }
  bn -= nb_first;
  const int KT = p.K >> 7;
  const int m_wg = bm * WGM;
  const int tile_base = DUAL ? bn * (WN * 2) + wn * 2 : bn * (WN * 4) + wn * 4;

  // Every global address below is a uniform base pointer plus a 32-bit byte
  // offset per lane (the launcher checks that the operands are smaller than
  // 4 GiB): one offset register instead of a 64-bit pointer pair per stream.
  const char* qwb = reinterpret_cast<const char*>(p.qw);
  const char* swb = reinterpret_cast<const char*>(p.sw);
  // DUAL: tiles 2 and 3 of the wave are the up projection's tiles of the channels of tiles 0 and 1
  const char* qwb2 = DUAL ? reinterpret_cast<const char*>(P.seg[1].qw) : qwb;
  const char* swb2 = DUAL ? reinterpret_cast<const char*>(P.seg[1].sw) : swb;
  uint32_t woff[4]; // slot index of this lane in tile nt at K step 0
#pragma unroll
  for (int nt = 0; nt < 4; nt++)
    woff[nt] = (uint32_t)(min(tile_base + (DUAL ? (nt & 1) : nt), p.tiles - 1) * KT * 64 + lane);

  // A tile (256 rows x 128 K, 64 KiB): 64 blocks of 4 rows x 256 B go from
  // global memory straight into LDS, one wave instruction per block (lane =
  // row r of the block, 16-byte chunk).  The LDS image of an instruction is
  // lane-linear, so the swizzle is applied on the global side: the lane at
  // position ch of row m fetches chunk ch ^ (m & 15).  Operand reads of one K
  // group (16 rows, same chunk) then fall on 16 different bank groups.
  //   LDS byte address of chunk ck of row m of row tile mt:
  //     mt*4096 + (m>>2)*1024 + (m&3)*256 + ((ck ^ m) & 15)*16
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(tl_lds); // LDS byte address of the buffers
  uint32_t rdb[4]; // byte offset of this lane's operand for step j (+ mt*4096): chunk ck = g*4 + j
  {
    const int m = lane & 15, g = lane >> 4;
#pragma unroll
    for (int j = 0; j < 4; j++)
      rdb[j] = (uint32_t)((m >> 2) * 1024 + (m & 3) * 256 + (((g * 4 + j) ^ m) & 15) * 16);
  }
  const char* xbase = reinterpret_cast<const char*>(p.x);
  // this wave's NBLK blocks: blk = wave*NBLK + i -> rows blk*4 + (lane>>4)
  const int rin = (lane >> 4);          // row inside the block
  const int ch = lane & 15;             // chunk position of this lane inside the row
  // source byte offset of block i at K step ks:
  //   row(i) * K * 2 + ((ch ^ m16(i)) & 15) * 16 + ks * 256, row(i) = m_wg + (wave*8 + i)*4 + rin,
  //   m16(i) = (i & 3)*4 + rin (wave*8 is a multiple of 4)
  const bool full = m_wg + WGM <= p.M; // uniform
  const uint32_t xrow0 = (uint32_t)((m_wg + wave * (NBLK * 4) + rin) * p.K) * 2u;
  const uint32_t blk_stride = (uint32_t)(4 * p.K) * 2u; // uniform
  auto load_a_one = [&](auto I, int ks, int buf) {
    constexpr int i = decltype(I)::value;
    const uint32_t sw = (uint32_t)((ch ^ ((i & 3) * 4 + rin)) & 15) * 16u;
    uint32_t off;
    if (full) {
      off = xrow0 + (uint32_t)i * blk_stride + sw + (uint32_t)ks * 256u;
    } else { // past the end: re-read the last row (never stored)
      const int row = min(m_wg + (wave * NBLK + i) * 4 + rin, p.M - 1);
      off = (uint32_t)(row * p.K) * 2u + sw + (uint32_t)ks * 256u;
    }
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xbase + (size_t)off),
                                     (__attribute__((address_space(3))) void*)(tl_lds + buf * ABUF + (wave * NBLK + i) * 1024),
                                     16, 0, 0);
  };
  auto load_a = [&](int ks, int buf) { static_for<0, NBLK>([&](auto I) { load_a_one(I, ks, buf); }); };
  // B of one K step: 4 tiles x 4 dwords (one per step j) and the scale factors
  uint32_t bc[4][4];
  float sc[4];
  i32x4 bnext[4];
  uint32_t snext[4];
  auto load_b = [&](int ks) {
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      const uint32_t slot = woff[nt] + (uint32_t)ks * 64u;
      bnext[nt] = *reinterpret_cast<const i32x4*>((nt < 2 ? qwb : qwb2) + (size_t)(slot * 16u));
      snext[nt] = *reinterpret_cast<const uint8_t*>((nt < 2 ? swb : swb2) + (size_t)slot);
    }
  };
  auto take_b = [&]() {
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
#pragma unroll
      for (int j = 0; j < 4; j++)
        bc[nt][j] = (uint32_t)bnext[nt][j];
      sc[nt] = e8m0_to_f32(snext[nt]);
    }
  };
  i32x4 bw[4][4]; // WBF16: [j][nt]
  auto load_bw = [&](int ks, int j) {
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      // native bf16 tiles: slot ((tile * KT + ks) * 4 + j) * 64 + lane, 16 bytes each
      const char* src = qwb + (size_t)(((woff[nt] - (uint32_t)lane) * 4u + (uint32_t)(ks * 4 + j) * 64u + (uint32_t)lane) * 16u);
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(bw[j][nt]) : "v"(src));
    }
  };

  f32x4 acc[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  load_a(0, 0);
  if constexpr (WBF16) {
#pragma unroll
    for (int j = 0; j < 4; j++)
      load_bw(0, j);
  } else {
    load_b(0);
  }
  __syncthreads();
  // One K step.  MORE: the next step's A tile is requested during this one, one block behind each of the first NBLK
  // MFMA groups (issued in one burst, a wave stands at its load instructions while the memory pipeline's queue
  // drains, and its MFMAs wait with it); it lands in the other buffer.
  auto step = [&](auto MORE, int ks) {
    constexpr bool more = decltype(MORE)::value;
    const int buf = ks & 1;
    if constexpr (!WBF16)
      take_b();
    // 4*MT operand reads per K step (q = j*MT + mt), kept RD ahead of the MFMAs
    // that consume them so the LDS latency is covered by 4*RD MFMAs
    const uint32_t abase = lds0 + (uint32_t)(buf * ABUF + wm * MT * 4096);
    constexpr int RD = 3; // operand reads in flight ahead of the MFMAs
    constexpr int NQ = 4 * MT;
    i32x4 ar[RD + 1];
    bf16x8 b[4];
    static_for<0, RD>([&](auto I) {
      constexpr int i = decltype(I)::value;
      lds_read_b128_async<(i % MT) * 4096>(ar[i], abase + rdb[i / MT]);
    });
    static_for<0, NQ>([&](auto Q) {
      constexpr int q = decltype(Q)::value;
      constexpr int j = q / MT, mt = q % MT;
      if constexpr (mt == 0 && WBF16) {
        // Step j's weights were requested a K step ago, behind group j * MT + MT - 1.  Behind them then: the later
        // steps' (4 each) and the blocks of A that K step still had to request (block d goes out behind group d);
        // in this K step, when it requests anything: the blocks of A behind the groups before this one and the
        // next K step's weights of the steps before j.
        constexpr int qj = j * MT + MT - 1;
        constexpr int younger = (3 - j) * 4 + (NBLK - 1 - qj > 0 ? NBLK - 1 - qj : 0) +
                                (more ? (j * MT < NBLK ? j * MT : NBLK) + j * 4 : 0);
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(bw[j][0]), "+v"(bw[j][1]), "+v"(bw[j][2]), "+v"(bw[j][3]) : "n"(younger));
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
          b[nt] = __builtin_bit_cast(bf16x8, bw[j][nt]);
      }
      if constexpr (mt == 0 && !WBF16) {
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
          b[nt] = tl_cvt_fp4x8(bc[nt][j], sc[nt]);
      }
      if constexpr (q + RD < NQ) {
        lds_read_b128_async<((q + RD) % MT) * 4096>(ar[(q + RD) % (RD + 1)], abase + rdb[(q + RD) / MT]);
        lds_wait_keep<RD>(ar[q % (RD + 1)]);
      } else {
        lds_wait_keep<NQ - 1 - q>(ar[q % (RD + 1)]);
      }
      const bf16x8 a = __builtin_bit_cast(bf16x8, ar[q % (RD + 1)]);
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[nt], acc[mt][nt], 0, 0, 0);
      if constexpr (more && q < NBLK)
        load_a_one(std::integral_constant<int, q>{}, ks + 1, buf ^ 1);
      if constexpr (WBF16) {
        if constexpr (more && mt == MT - 1)
          load_bw(ks + 1, j); // the MFMAs that read step j's registers have been issued
      } else {
        if constexpr (more && q == NQ / 2 - 1)
          load_b(ks + 1); // dwords of steps 0 and 1 of the current B are dead by now
      }
    });
    if constexpr (WBF16 && more) {
      // this wave's loads into LDS have landed -- behind the last of them went out the next K step's weights of
      // every step j whose last group is not before that block's -- then everybody's; a bare barrier, see above
      constexpr int after = 4 * ((MT - 1 >= NBLK - 1) + (2 * MT - 1 >= NBLK - 1) + (3 * MT - 1 >= NBLK - 1) + (4 * MT - 1 >= NBLK - 1));
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(after) : "memory");
    } else {
      __syncthreads(); // waits for this wave's direct-to-LDS loads, then for everybody's
    }
  };
  for (int ks = 0; ks + 1 < KT; ks++)
    step(std::true_type{}, ks);
  step(std::false_type{}, KT - 1);
  // every wave has left the main loop (barrier above): LDS is free for the epilogue staging
  if (DUAL)
    big_epilogue_dual<MT>(p, P.seg[1], acc, reinterpret_cast<float*>(tl_lds) + wave * 64 * EP_LD, m_wg + wm * (MT * 16),
                          tile_base);
  else
    big_epilogue<MT>(p, acc, reinterpret_cast<float*>(tl_lds) + wave * 64 * EP_LD, m_wg + wm * (MT * 16), tile_base);
}

template <int MT, bool DUAL, int WM, int WN>
__global__ void __launch_bounds__(WM * WN * 64, WM * WN == 4 ? 2 : 1)
big_mxfp4_kernel(const BigParams P) {
  big_gemm_body<MT, DUAL, WM, WN, false>(P);
}

template <int MT, int WM, int WN>
__global__ void __launch_bounds__(WM * WN * 64, WM * WN == 4 ? 2 : 1)
big_bf16_kernel(const BigParams P) {
  big_gemm_body<MT, false, WM, WN, true>(P);
}

// ---------------------------------------------------------------------------
// Large-M QINT8 (W8A8, 256-wide blocks): 128 x 256 workgroup tile, 8 waves
// (2 x 4), wave tile 64 x 64, K step 256 = one scale block.
// What bounds int8 at this size is operand delivery and the fold, not the
// MFMA: weights are 4x the bytes of MXFP4 per MAC, the MFMA runs at twice the
// bf16 rate, and every block's int32 sums have to be converted, scaled by
// sa[m] * sw[n] and added to the fp32 sums: 3 vector instructions per output
// and block, 3 per MFMA.  Measured on this part, an int8 MFMA holds its SIMD's
// vector issue for about 8 cycles and any other vector instruction for 4,
// whichever wave they come from (16.5 / 17.5 / 18 / 21.5 / 25.5 cycles per MFMA
// with 0 / 1 / 2 / 3 / 4 independent fp32 instructions behind each), so the
// fold alone caps the MFMA busy fraction near 0.73.  So:
//   * BOTH operands go from global memory straight into LDS (no staging
//     registers, nothing for the compiler to wait on before the barrier) and
//     every weight tile is fetched once per workgroup instead of once per wave
//     row.  A: int8 rows, 256 B per row and step, the layout, swizzle and
//     operand reads of the MXFP4 kernel above (operand of MFMA step j = chunk
//     j*4 + g of the row), two buffers.  B: native 1 KiB tiles (lane-linear =
//     operand order), 16 tiles x 4 K tiles = 64 KiB, ONE buffer: at the start
//     of a step every wave copies its 16 operands into registers, a barrier
//     frees the buffer and the next step's tiles stream in during the MFMAs.
//   * The MFMAs of a step run row tile by row tile (all of K for 16 rows, then
//     the next 16), into one of two small sets of int32 sums, and the fold of
//     row tile mt sits between the first and the second MFMA group of row tile
//     mt + 1: vector and matrix work overlap inside a wave, and the two waves
//     of a SIMD do not fold at the same moment.  The first MFMA of a row tile
//     starts from a zero operand.
//   * Activation scales reach the waves through LDS, requested two steps ahead.
// LDS: A 2 x 32 KiB | B 64 KiB | scales 2 KiB (the epilogue staging reuses it).
// ---------------------------------------------------------------------------
template <int N>
__device__ __forceinline__ void lds_wait_keep16(i32x4 (&b)[4][4]) {
  asm volatile("s_waitcnt lgkmcnt(%16)"
               : "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[0][2]), "+v"(b[0][3]), "+v"(b[1][0]), "+v"(b[1][1]), "+v"(b[1][2]),
                 "+v"(b[1][3]), "+v"(b[2][0]), "+v"(b[2][1]), "+v"(b[2][2]), "+v"(b[2][3]), "+v"(b[3][0]), "+v"(b[3][1]),
                 "+v"(b[3][2]), "+v"(b[3][3])
               : "n"(N));
}

// MT = row tiles of 16 per wave: 4 (workgroup 128 x 256) or 2 (64 x 256, for launches that leave CUs empty).
template <int MT>
__device__ __forceinline__ void big_qint8_body(const BigParams& P) {
  constexpr int WGM = MT * 32, ABUF = WGM * 256, BBUF = 64 * 1024;
  extern __shared__ __align__(16) uint8_t tl_lds[];
  uint8_t* b_lds = tl_lds + 2 * ABUF;
  float* sa_s = reinterpret_cast<float*>(tl_lds + 2 * ABUF + BBUF); // [4][128]: scales of steps ks .. ks+2 (mod 4)
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int MB = (P.seg[0].M + WGM - 1) / WGM;
  int bm, bn;
  tile_of_block(MB, P.nb0[P.n_seg], bm, bn);
  // several GEMMs over one activation (fused q/k/v) share the launch: pick this block's with uniform selects
  TiledParams p = P.seg[0];
  int nb_first = 0;
#pragma unroll
  for (int i = 1; i < TPPX_MAX_SEGS; i++)
    if (i < P.n_seg && bn >= P.nb0[i]) {
      p = P.seg[i];
      nb_first = P.nb0[i];
    }
  bn -= nb_first;
  const int KS = p.K >> 8;   // K steps = scale blocks
  const int KT64 = p.K >> 6; // native tiles along K
  const int m_wg = bm * WGM;
  const int tile_base = bn * 16 + wn * 4;

  const float* swp = reinterpret_cast<const float*>(p.sw);
  uint32_t soff[4];
#pragma unroll
  for (int nt = 0; nt < 4; nt++)
    soff[nt] = (uint32_t)(min(tile_base + nt, p.tiles - 1) * KS * 16 + (lane & 15));
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(tl_lds);
  uint32_t rdb[4];
  {
    const int m = lane & 15, g = lane >> 4;
#pragma unroll
    for (int j = 0; j < 4; j++)
      rdb[j] = (uint32_t)((m >> 2) * 1024 + (m & 3) * 256 + (((j * 4 + g) ^ m) & 15) * 16);
  }
  const char* xbase = reinterpret_cast<const char*>(p.xq);
  const int rin = lane >> 4, ch = lane & 15;
  const bool full = m_wg + WGM <= p.M;
  const uint32_t xrow0 = (uint32_t)((m_wg + wave * (MT * 4) + rin) * p.K);
  const uint32_t blk_stride = (uint32_t)(4 * p.K);
  auto load_a_one = [&](auto I, int ks, int buf) {
    constexpr int i = decltype(I)::value;
    // row of this block inside its 16-row tile: the wave's first block is a multiple of 4 only with four row tiles
    const uint32_t sw = (uint32_t)((ch ^ (((wave * MT + i) & 3) * 4 + rin)) & 15) * 16u;
    uint32_t off;
    if (full) {
      off = xrow0 + (uint32_t)i * blk_stride + sw + (uint32_t)ks * 256u;
    } else {
      const int row = min(m_wg + (wave * MT + i) * 4 + rin, p.M - 1);
      off = (uint32_t)(row * p.K) + sw + (uint32_t)ks * 256u;
    }
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xbase + (size_t)off),
                                     (__attribute__((address_space(3))) void*)(tl_lds + buf * ABUF + (wave * MT + i) * 1024),
                                     16, 0, 0);
  };
  auto load_a = [&](int ks, int buf) { static_for<0, MT>([&](auto I) { load_a_one(I, ks, buf); }); };
  // B of step ks: this wave brings tiles 2*wave, 2*wave + 1 of the 16, all four K tiles; LDS slot (tile*4 + kt) KiB
  const char* qwb = reinterpret_cast<const char*>(p.qw);
  uint32_t bsrc[2];
#pragma unroll
  for (int i = 0; i < 2; i++)
    bsrc[i] = (uint32_t)(min(bn * 16 + wave * 2 + i, p.tiles - 1) * KT64 * 64 + lane);
  auto load_b_one = [&](auto I, int ks) {
    constexpr int i = decltype(I)::value >> 2, kt = decltype(I)::value & 3;
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void*)(qwb + (size_t)((bsrc[i] + (uint32_t)(ks * 4 + kt) * 64u) * 16u)),
        (__attribute__((address_space(3))) void*)(b_lds + ((wave * 2 + i) * 4 + kt) * 1024), 16, 0, 0);
  };
  auto load_b = [&](int ks) { static_for<0, 8>([&](auto I) { load_b_one(I, ks); }); };
  // activation scales: thread t < 128 carries the scale of row t for the step two ahead
  const float* sarow = p.sa + (int64_t)min(m_wg + (tid & 127), p.M - 1) * KS;
  float sareg = 0.f;
  float swv[4], swn[4];

  f32x4 facc[MT][4];
  i32x4 iacc[2][4]; // block sums of the row tile in flight and of the one being folded
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      facc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      iacc[i][nt] = i32x4{0, 0, 0, 0};

  load_a(0, 0);
  load_b(0);
#pragma unroll
  for (int nt = 0; nt < 4; nt++)
    swn[nt] = swp[soff[nt]];
  if (tid < WGM) {
    sa_s[tid] = sarow[0];
    if (KS > 1)
      sa_s[128 + tid] = sarow[1];
    sareg = KS > 2 ? sarow[2] : 0.f;
  }
  __syncthreads();
  const uint32_t bwave = lds0 + (uint32_t)(2 * ABUF + wn * 16 * 1024) + (uint32_t)lane * 16u; // this wave's 4 tiles
  // One K step.  MORE: the next step's tiles are requested one wave instruction at a time behind the MFMA groups
  // (in one burst, a wave stands at its load instructions while the memory pipeline's queue drains).
  auto step = [&](auto MORE, int ks) {
    constexpr bool more = decltype(MORE)::value;
    const int buf = ks & 1;
    // this step's weight operands: LDS -> registers, then the buffer is free for the next step's tiles
    i32x4 bq[4][4]; // [tile][MFMA step j]
    static_for<0, 16>([&](auto I) {
      constexpr int i = decltype(I)::value;
      lds_read_b128_async<i * 1024>(bq[i >> 2][i & 3], bwave);
    });
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      swv[nt] = swn[nt];
    if (tid < WGM && ks + 2 < KS) {
      sa_s[((ks + 2) & 3) * 128 + tid] = sareg; // loaded two steps ago
      sareg = ks + 3 < KS ? sarow[ks + 3] : 0.f;
    }
    lds_wait_keep16<0>(bq);
    __syncthreads();
    if constexpr (more) {
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        swn[nt] = swp[soff[nt] + (uint32_t)(ks + 1) * 16u];
    }
    const uint32_t abase = lds0 + (uint32_t)(buf * ABUF + wm * MT * 4096);
    const float* sab = sa_s + (ks & 3) * 128 + wm * (MT * 16) + (lane >> 4) * 4;
    auto fold = [&](auto MTI) { // facc += int32 sum * (sa[row] * sw[channel]) for row tile mt
      constexpr int mt = decltype(MTI)::value;
      const f32x4 sav = *reinterpret_cast<const f32x4*>(sab + mt * 16);
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          facc[mt][nt][r] = fmaf((float)iacc[mt & 1][nt][r], sav[r] * swv[nt], facc[mt][nt][r]);
    };
    // activation operands in order q = mt*4 + j, RD ahead of their use
    constexpr int RD = 3, NQ = 4 * MT;
    i32x4 ar[RD + 1];
    static_for<0, RD>([&](auto I) {
      constexpr int i = decltype(I)::value;
      lds_read_b128_async<(i / 4) * 4096>(ar[i], abase + rdb[i % 4]);
    });
    static_for<0, NQ>([&](auto Q) {
      constexpr int q = decltype(Q)::value;
      constexpr int mt = q / 4, j = q % 4;
      if constexpr (q + RD < NQ) {
        lds_read_b128_async<((q + RD) / 4) * 4096>(ar[(q + RD) % (RD + 1)], abase + rdb[(q + RD) % 4]);
        lds_wait_keep<RD>(ar[q % (RD + 1)]);
      } else {
        lds_wait_keep<NQ - 1 - q>(ar[q % (RD + 1)]);
      }
      const i32x4 a = ar[q % (RD + 1)];
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        iacc[mt & 1][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bq[nt][j], j == 0 ? i32x4{0, 0, 0, 0} : iacc[mt & 1][nt], 0, 0, 0);
      if constexpr (more && q < 8)
        load_b_one(std::integral_constant<int, q>{}, ks + 1);
      // the MT blocks of A behind the groups after the weight tiles' (with two row tiles there are only 8 groups: behind the last MT of them)
      constexpr int qa = NQ >= 8 + MT ? 8 : NQ - MT;
      if constexpr (more && q >= qa && q < qa + MT)
        load_a_one(std::integral_constant<int, q - qa>{}, ks + 1, buf ^ 1);
      if constexpr (j == 0 && mt > 0)
        fold(std::integral_constant<int, mt - 1>{}); // the previous row tile, under this row tile's MFMAs
    });
    fold(std::integral_constant<int, MT - 1>{});
    __syncthreads();
  };
  for (int ks = 0; ks + 1 < KS; ks++)
    step(std::true_type{}, ks);
  step(std::false_type{}, KS - 1);
  big_epilogue<MT>(p, facc, reinterpret_cast<float*>(tl_lds) + wave * 64 * EP_LD, m_wg + wm * (MT * 16), tile_base);
}

__global__ void __launch_bounds__(512)
big_qint8_kernel(const BigParams P) {
  big_qint8_body<4>(P);
}

__global__ void __launch_bounds__(512)
big_qint8_small_kernel(const BigParams P) {
  big_qint8_body<2>(P);
}

// the large-M kernel addresses its operands with 32-bit byte offsets
// ---------------------------------------------------------------------------
// Large-M MXFP4 weights x MXFP8 activations on the block-scaled MFMA
// (v_mfma_scale_f32_16x16x128_f8f6f4): the weights' E2M1 codes and E8M0 scales
// are the instruction's operands as they lie in the native tiles -- nothing is
// expanded -- and the activations arrive quantised in operand order
// (quant_act_mxfp8_kernel).  Not the reference's arithmetic (its activations
// stay bf16): an opt-in (TPPX_FLAG_ACT_FP8).
// Workgroup tile (MT*32) x 256, 8 waves (2 x 4), wave tile (MT*16) x 64 =
// 4*MT MFMAs of K = 128 per step; MT = 8 (256 rows) or 4 (128 rows).
// Everything a step needs -- both operands AND both sets of scale bytes -- goes
// from global memory straight into LDS (1 KiB per wave instruction for the
// operands: a native weight tile, half an activation tile, lane-linear on both
// sides, so operand reads are conflict-free 16-byte reads; 256 B per wave
// instruction for scales), NB - 1 steps ahead in a ring of NB stages.  All
// loads of the loop being of this one kind, they complete in issue order and
// the wait at the top of a step is a partial one (the younger stages stay in
// flight); one barrier per step.
// ---------------------------------------------------------------------------
typedef int i32x8 __attribute__((ext_vector_type(8)));

template <int N>
__device__ __forceinline__ void lds_wait_keep2(i32x4& a, i32x4& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}

template <int MT>
struct Fp8Geom {
  static constexpr int NB = MT == 8 ? 3 : 4;        // stages in the ring
  static constexpr int A_BYTES = MT * 4096;         // 2*MT row tiles of 2 KiB
  static constexpr int B_OFF = A_BYTES;             // 16 weight tiles of 1 KiB
  static constexpr int SA_OFF = B_OFF + 16384;      // MT/2 groups of 64 rows x 256 B
  static constexpr int SB_OFF = SA_OFF + MT * 128;  // 16 tiles x 64 B
  static constexpr int STAGE = SB_OFF + 1024;
  static constexpr int LPS = MT / 2 + 2 + 1;        // loads per wave and stage: A halves, weight tiles, one of scales
};

// DUAL: the gate/up pair as in big_mxfp4_kernel: 128 output channels per workgroup, the 16 weight tiles of a stage are
// 4 x (2 gate tiles, the 2 up tiles of the same channels), one group per wave column; silu(gate) * up in the epilogue.
template <int MT, bool DUAL>
__global__ void __launch_bounds__(512)
big_fp8_kernel(const BigParams P) {
  using G = Fp8Geom<MT>;
  constexpr int NB = G::NB, STAGE = G::STAGE, LPS = G::LPS;
  extern __shared__ __align__(16) uint8_t tl_lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int MB = (P.seg[0].M + MT * 32 - 1) / (MT * 32);
  int bm, bn;
  tile_of_block(MB, P.nb0[P.n_seg], bm, bn);
  TiledParams p = P.seg[0];
  int nb_first = 0;
  if (!DUAL) {
#pragma unroll
    for (int i = 1; i < TPPX_MAX_SEGS; i++)
      if (i < P.n_seg && bn >= P.nb0[i]) {
        p = P.seg[i];
        nb_first = P.nb0[i];
      }
  }
  bn -= nb_first;
  const int KT = p.K >> 7;
  const int m_wg = bm * (MT * 32);
  const int tile_base = DUAL ? bn * 8 + wn * 2 : bn * 16 + wn * 4;
  // weight tile behind slot t (0..15) of a stage, and whether it is the up projection's (DUAL)
  auto slot_tile = [&](int t) { return DUAL ? bn * 8 + (t >> 2) * 2 + (t & 1) : bn * 16 + t; };
  auto slot_up = [&](int t) { return DUAL && (t & 2) != 0; };
  const int Q = (p.M + 63) >> 6; // 64-row groups of the quantised activations (rows padded to 64)

  // this wave's share of a stage: MT/2 activation half tiles, 2 weight tiles, one 256-byte piece of scales
  const char* xqb = reinterpret_cast<const char*>(p.xq);
  const char* qwb = reinterpret_cast<const char*>(p.qw);
  const char* a_src[MT / 2];
#pragma unroll
  for (int i = 0; i < MT / 2; i++) {
    const int j = wave * (MT / 2) + i; // half tile j of the 4*MT: row tile j >> 1, half j & 1
    a_src[i] = xqb + ((size_t)min(bm * (MT * 2) + (j >> 1), Q * 4 - 1) * KT * 2 + (j & 1)) * 1024 + (size_t)lane * 16;
  }
  const char* b_src[2];
#pragma unroll
  for (int i = 0; i < 2; i++)
    b_src[i] = (slot_up(wave * 2 + i) ? reinterpret_cast<const char*>(P.seg[1].qw) : qwb) +
               ((size_t)min(slot_tile(wave * 2 + i), p.tiles - 1) * KT) * 1024 + (size_t)lane * 16;
  const char* s_src;
  int s_dst, s_stride;
  if (wave < MT / 2) { // activation scales of 64-row group `wave`: [Q][KT][64 lanes][4 row tiles]
    s_src = reinterpret_cast<const char*>(p.sa) + (size_t)min(bm * (MT / 2) + wave, Q - 1) * KT * 256 + (size_t)lane * 4;
    s_dst = G::SA_OFF + wave * 256;
    s_stride = 256;
  } else { // weight scales of tiles 4i .. 4i+3: native [tile][KT][64]
    int i = wave - MT / 2;
    if (i >= 4)
      i -= 2; // 128-row form: waves 6, 7 repeat what 4, 5 fetch, so that every wave issues LPS loads per stage
    const int t = i * 4 + (lane >> 4);
    s_src = reinterpret_cast<const char*>(slot_up(t) ? P.seg[1].sw : p.sw) + (size_t)min(slot_tile(t), p.tiles - 1) * KT * 64 +
            (size_t)(lane & 15) * 4;
    s_dst = G::SB_OFF + i * 256;
    s_stride = 64;
  }
  // load number I (of LPS) of this wave's share of a stage
  auto dma_one = [&](auto I, int ks, int buf) {
    constexpr int i = decltype(I)::value;
    uint8_t* base = tl_lds + buf * STAGE;
    if constexpr (i < MT / 2)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_src[i] + (size_t)ks * 2048),
                                       (__attribute__((address_space(3))) void*)(base + (wave * (MT / 2) + i) * 1024), 16, 0, 0);
    else if constexpr (i < MT / 2 + 2)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(b_src[i - MT / 2] + (size_t)ks * 1024),
                                       (__attribute__((address_space(3))) void*)(base + G::B_OFF + (wave * 2 + i - MT / 2) * 1024), 16, 0, 0);
    else
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(s_src + (size_t)ks * s_stride),
                                       (__attribute__((address_space(3))) void*)(base + s_dst), 4, 0, 0);
  };
  auto dma = [&](int ks, int buf) { static_for<0, LPS>([&](auto I) { dma_one(I, ks, buf); }); };

  f32x4 acc[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint32_t lds0 = (uint32_t)(uintptr_t)tl_lds;
#pragma unroll
  for (int s = 0; s < NB - 1; s++)
    if (s < KT)
      dma(s, s);
  int buf = 0;
  // One K step.  DMA: the loads of stage ks + NB - 1 are issued one at a time behind the MFMA groups of the step
  // (issued in one burst at the top, a wave stands at its load instructions while the memory pipeline's queue
  // drains, and its MFMAs wait with it).
  auto step = [&](auto DMA, int ks) {
    constexpr bool with_dma = decltype(DMA)::value;
    // stage ks has landed for this wave (the NB - 2 younger ones may still be in flight) ...
    if (with_dma || ks + NB - 2 < KT)
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"(LPS * (NB - 2)) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    // ... and for every wave; nobody still reads the stage of step ks - 1, which the next loads overwrite
    asm volatile("s_barrier" : : : "memory");
    const int nbuf = buf == 0 ? NB - 1 : buf - 1;
    const uint8_t* base = tl_lds + buf * STAGE;
    i32x4 bw[4];
    int sbv[4];
    uint32_t sav[MT / 4];
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      bw[nt] = *reinterpret_cast<const i32x4*>(base + G::B_OFF + (wn * 4 + nt) * 1024 + lane * 16);
      sbv[nt] = base[G::SB_OFF + (wn * 4 + nt) * 64 + lane];
    }
#pragma unroll
    for (int q = 0; q < MT / 4; q++)
      sav[q] = *reinterpret_cast<const uint32_t*>(base + G::SA_OFF + (wm * (MT / 4) + q) * 256 + lane * 4);
    // activation operands: the two halves of row tile mt, read two row tiles ahead of the MFMAs that use them
    const uint32_t abase = lds0 + (uint32_t)(buf * STAGE + wm * MT * 2048 + lane * 16);
    i32x4 alo[3], ahi[3];
    static_for<0, 2>([&](auto I) {
      constexpr int i = decltype(I)::value;
      lds_read_b128_async<i * 2048>(alo[i], abase);
      lds_read_b128_async<i * 2048 + 1024>(ahi[i], abase);
    });
    static_for<0, MT>([&](auto I) {
      constexpr int mt = decltype(I)::value;
      if constexpr (mt + 2 < MT) {
        lds_read_b128_async<(mt + 2) * 2048>(alo[(mt + 2) % 3], abase);
        lds_read_b128_async<(mt + 2) * 2048 + 1024>(ahi[(mt + 2) % 3], abase);
        lds_wait_keep2<4>(alo[mt % 3], ahi[mt % 3]);
      } else {
        lds_wait_keep2<(MT - 1 - mt) * 2>(alo[mt % 3], ahi[mt % 3]);
      }
      const i32x4 lo = alo[mt % 3], hi = ahi[mt % 3];
      const i32x8 a = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      const int sa = (int)((sav[mt >> 2] >> ((mt & 3) * 8)) & 0xffu);
#pragma unroll
      for (int nt = 0; nt < 4; nt++) {
        const i32x8 b = i32x8{bw[nt][0], bw[nt][1], bw[nt][2], bw[nt][3], 0, 0, 0, 0};
        acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[mt][nt], 0 /* A: E4M3 */,
                                                                       4 /* B: E2M1 */, 0, sa, 0, sbv[nt]);
      }
      if constexpr (with_dma) {
        // LPS loads over MT slots (LPS <= MT + 1: the last slot takes the remainder)
        if constexpr (mt < LPS)
          dma_one(std::integral_constant<int, mt>{}, ks + NB - 1, nbuf);
        if constexpr (mt == MT - 1)
          static_for<MT, (LPS > MT ? LPS : MT)>([&](auto J) { dma_one(J, ks + NB - 1, nbuf); });
      }
    });
    buf = buf == NB - 1 ? 0 : buf + 1;
  };
  int ks = 0;
  for (; ks + NB - 1 < KT; ks++)
    step(std::true_type{}, ks);
  for (; ks < KT; ks++)
    step(std::false_type{}, ks);
  __syncthreads(); // every wave has left the main loop: LDS is free for the epilogue staging
  if (DUAL)
    big_epilogue_dual<MT>(p, P.seg[1], acc, reinterpret_cast<float*>(tl_lds) + wave * 64 * EP_LD, m_wg + wm * (MT * 16),
                          tile_base);
  else
    big_epilogue<MT>(p, acc, reinterpret_cast<float*>(tl_lds) + wave * 64 * EP_LD, m_wg + wm * (MT * 16), tile_base);
}

// cost of a full round of 128 x 512 workgroups relative to one of 256 x 256 (measured)
constexpr double BIG_WIDE_COST = 0.97;

static bool big_fits(const TiledParams& p) {
  return (int64_t)p.M * p.K * 2 < ((int64_t)1 << 32) && (int64_t)p.tiles * 8 * p.K < ((int64_t)1 << 32);
}

bool tiled_mxfp4_takes_groups(const TiledParams& p) {
  return p.M >= big_min_rows() && big_fits(p);
}

template <int MT, bool DUAL, int WM, int WN>
static hipError_t big_launch(const BigParams& P, int wgs, hipStream_t stream) {
  // epilogue staging per wave; >= the two A buffers
  const size_t lds = (size_t)WM * WN * 64 * EP_LD * sizeof(float);
  static_assert((size_t)WM * WN * 64 * EP_LD * sizeof(float) >= (size_t)2 * MT * 16 * WM * 256, "LDS plan");
  TPPX_PLAN_ONLY((big_mxfp4_kernel<MT, DUAL, WM, WN>), dim3(wgs), dim3(WM * WN * 64), lds);
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(big_mxfp4_kernel<MT, DUAL, WM, WN>), lds); e != hipSuccess)
    return e;
  big_mxfp4_kernel<MT, DUAL, WM, WN><<<dim3(wgs), dim3(WM * WN * 64), lds, stream>>>(P);
  return hipGetLastError();
}

template <int MT, int WM, int WN>
static hipError_t big_bf16_launch(const BigParams& P, int wgs, hipStream_t stream) {
  const size_t lds = (size_t)WM * WN * 64 * EP_LD * sizeof(float);
  static_assert((size_t)WM * WN * 64 * EP_LD * sizeof(float) >= (size_t)2 * MT * 16 * WM * 256, "LDS plan");
  TPPX_PLAN_ONLY((big_bf16_kernel<MT, WM, WN>), dim3(wgs), dim3(WM * WN * 64), lds);
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(big_bf16_kernel<MT, WM, WN>), lds); e != hipSuccess)
    return e;
  big_bf16_kernel<MT, WM, WN><<<dim3(wgs), dim3(WM * WN * 64), lds, stream>>>(P);
  return hipGetLastError();
}

// dual: t[0] = gate, t[1] = up (equal shapes, n == 2); y[m][n] = silu(gate) * up goes to t[1].y
hipError_t launch_tiled_mxfp4_group(const TiledParams* t, int n, hipStream_t stream, bool dual) {
  if (dual && (n != 2 || t[0].tiles != t[1].tiles || t[0].K != t[1].K || t[0].M != t[1].M || t[0].x != t[1].x))
    return hipErrorInvalidValue;
  // channel blocks of the launch when a workgroup owns `tpw` channel tiles (of each projection for the pair)
  auto blocks = [&](int tpw) {
    int nb = 0;
    for (int i = 0; i < (dual ? 1 : n); i++)
      nb += (t[i].tiles + tpw - 1) / tpw;
    return nb;
  };
  const int nb4 = blocks(dual ? 8 : 16), nb8 = blocks(dual ? 16 : 32); // 4 or 8 wave columns
  const int MB8 = (t[0].M + 255) / 256, MB4 = (t[0].M + 127) / 128;
  // Workgroup tile.  256 x 256 (8 waves, one per CU) or 128 x 512 (8 waves, one per CU) when their rounds of 256
  // workgroups are full; 128 x 256 (4 waves, two per CU, 512 at a time) costs a few percent more per round but its
  // workgroups are half the size, so a last partial round costs less (q/k/v with 10240 channels at M = 2048: 320
  // workgroups of 256 x 256 are 2 rounds, 640 of 128 x 256 are 1.25).  Costs in units of one full round of 256 x 256.
  auto rounds = [](int wgs) { return (double)((wgs + 255) / 256); };
  const int w4 = MB4 * nb4;
  const double cost[3] = {rounds(MB8 * nb4), w4 <= 256 ? 0.6 : 1.05 * (w4 <= 512 ? 1.0 : w4 / 512.0),
                          BIG_WIDE_COST * rounds(MB4 * nb8)};
  int shape = 0;
  for (int i = 1; i < 3; i++)
    if (cost[i] < cost[shape])
      shape = i;
  const int env_shape = env_int("TPPX_TILED_BIG_TILE", 0); // 1 = 256 x 256, 2 = 128 x 256, 3 = 128 x 512
  if (env_shape >= 1 && env_shape <= 3)
    shape = env_shape - 1;
  // Launches that would leave half the CUs empty with 128 x 256 workgroups: 64 x 128 workgroups of four waves (32 x 64
  // each) instead, four times as many (the same sums in the same order: the same bits; 4096 x 4096 at 256 rows
  // 50 -> 28 us, 4096 x 11008 at 512 rows 124 -> 79 us; beyond 128 such workgroups the small ones lose)
  const bool small = shape == 1 && MB4 * nb4 <= 128 && env_int("TPPX_TILED_SMALL", 1) != 0 && env_shape == 0;
  const int tpw = small ? (dual ? 4 : 8) : (shape == 2 ? 8 : 4) * (dual ? 2 : 4);
  BigParams P;
  memset(&P, 0, sizeof(P));
  int nb = 0;
  for (int i = 0; i < n; i++) {
    P.seg[i] = t[i];
    P.nb0[i] = nb;
    nb += (t[i].tiles + tpw - 1) / tpw;
  }
  if (dual) {
    nb = (t[0].tiles + tpw - 1) / tpw;
    P.nb0[1] = nb;
  }
  for (int i = n; i <= TPPX_MAX_SEGS; i++)
    P.nb0[i] = nb;
  P.n_seg = n;
  {
    // XCD rectangles: the split that moves the fewest bytes from memory into the L2s (activations: rows x K bf16 per
    // row block, fetched by 8 / xm XCDs... every XCD fetches 1/xm of them; weights 0.53 B per element, xm/8 each)
    const int MBs = small ? (t[0].M + 63) / 64 : shape == 0 ? MB8 : MB4;
    const double a_bytes = (double)t[0].M * t[0].K * 2.0, w_bytes = (dual ? 2.0 : 1.0) * nb * tpw * 16.0 * t[0].K * 0.53;
    double best = 1e300;
    P.xm = 1;
    for (int xm = 1; xm <= 4; xm *= 2)
      if (MBs % xm == 0 && nb % (8 / xm) == 0) {
        const double fill = 8.0 * (a_bytes / xm + w_bytes * xm / 8.0);
        if (fill < best) {
          best = fill;
          P.xm = xm;
        }
      }
    const int env_xm = env_int("TPPX_TILED_XCD_M", 0);
    if ((env_xm == 1 || env_xm == 2 || env_xm == 4) && MBs % env_xm == 0 && nb % (8 / env_xm) == 0)
      P.xm = env_xm;
  }
  if (shape == 2)
    return dual ? big_launch<8, true, 1, 8>(P, MB4 * nb, stream) : big_launch<8, false, 1, 8>(P, MB4 * nb, stream);
  // 128 x 256 workgroups that do not fill the CUs (at most one each): eight waves of 64 x 64 instead of four of
  // 128 x 64 -- two waves per SIMD, so that one wave's waits are another's issue slots (the same sums in the same
  // order: the same bits; 4096 x 4096 at 192-1024 rows 63-70 -> 49-57 us)
  if (small)
    return dual ? big_launch<2, true, 2, 2>(P, ((t[0].M + 63) / 64) * nb, stream)
                : big_launch<2, false, 2, 2>(P, ((t[0].M + 63) / 64) * nb, stream);
  if (shape == 1 && MB4 * nb <= 256 && env_int("TPPX_TILED_W8", 1) != 0)
    return dual ? big_launch<4, true, 2, 4>(P, MB4 * nb, stream) : big_launch<4, false, 2, 4>(P, MB4 * nb, stream);
  if (shape == 1)
    return dual ? big_launch<8, true, 1, 4>(P, MB4 * nb, stream) : big_launch<8, false, 1, 4>(P, MB4 * nb, stream);
  return dual ? big_launch<8, true, 2, 4>(P, MB8 * nb, stream) : big_launch<8, false, 2, 4>(P, MB8 * nb, stream);
}

// MXFP4 weights x MXFP8 activations (t[i].xq = quantised activations in operand order, t[i].sa = their scale bytes)
template <int MT, bool DUAL>
static hipError_t fp8_launch(const BigParams& P, int wgs, hipStream_t stream) {
  const size_t ep = 8 * 64 * EP_LD * sizeof(float); // epilogue staging
  const size_t lds = std::max(ep, (size_t)Fp8Geom<MT>::NB * Fp8Geom<MT>::STAGE);
  TPPX_PLAN_ONLY((big_fp8_kernel<MT, DUAL>), dim3(wgs), dim3(512), lds);
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(big_fp8_kernel<MT, DUAL>), lds); e != hipSuccess)
    return e;
  big_fp8_kernel<MT, DUAL><<<dim3(wgs), dim3(512), lds, stream>>>(P);
  return hipGetLastError();
}

// dual: the gate/up pair (t[0] = gate, t[1] = up, equal shapes); silu(gate) * up goes to t[1].y
hipError_t launch_tiled_mxfp4_fp8_group(const TiledParams* t, int n, hipStream_t stream, bool dual) {
  if (dual && (n != 2 || t[0].tiles != t[1].tiles || t[0].K != t[1].K || t[0].M != t[1].M || t[0].xq != t[1].xq))
    return hipErrorInvalidValue;
  BigParams P;
  memset(&P, 0, sizeof(P));
  int nb = 0;
  for (int i = 0; i < n; i++) {
    P.seg[i] = t[i];
    P.nb0[i] = nb;
    nb += (t[i].tiles + 15) / 16;
  }
  if (dual) {
    nb = (t[0].tiles + 7) / 8; // 128 output channels (gate and up of each) per workgroup
    P.nb0[1] = nb;
  }
  for (int i = n; i <= TPPX_MAX_SEGS; i++)
    P.nb0[i] = nb;
  P.n_seg = n;
  // 256-row tiles unless 128-row ones fill the last round of workgroups (256 CUs, one workgroup each) better
  const int MB8 = (t[0].M + 255) / 256, MB4 = (t[0].M + 127) / 128;
  auto rounds = [](int wgs) { return (wgs + 255) / 256; };
  const double cost8 = rounds(MB8 * nb), cost4 = 0.5 * 1.15 * rounds(MB4 * nb);
  int mt = cost4 < cost8 ? 4 : 8;
  const int env_mt = env_int("TPPX_FP8_BIG_MT", 0);
  if (env_mt == 4 || env_mt == 8)
    mt = env_mt;
  if (mt == 4)
    return dual ? fp8_launch<4, true>(P, MB4 * nb, stream) : fp8_launch<4, false>(P, MB4 * nb, stream);
  return dual ? fp8_launch<8, true>(P, MB8 * nb, stream) : fp8_launch<8, false>(P, MB8 * nb, stream);
}

hipError_t launch_tiled_mxfp4(const TiledParams& p, hipStream_t stream) {
  if (tiled_mxfp4_takes_groups(p))
    return launch_tiled_mxfp4_group(&p, 1, stream);
  const int MB = (p.M + 127) / 128, NB = (p.tiles + 7) / 8;
  const size_t lds = 2 * 2048 * 16;
  TPPX_PLAN_ONLY(tiled_mxfp4_kernel, dim3(MB * NB), dim3(256), lds);
  if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(tiled_mxfp4_kernel), lds); e != hipSuccess)
    return e;
  tiled_mxfp4_kernel<<<dim3(MB * NB), dim3(256), lds, stream>>>(p);
  return hipGetLastError();
}

// silu(gate) * up over two bf16 tiles that already hold bias + dot (see the gate/up group launch)
__global__ void __launch_bounds__(256)
silu_mul_kernel(const uint16_t* __restrict__ gate, uint16_t* __restrict__ y, int64_t n8) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    const uint4 g = reinterpret_cast<const uint4*>(gate)[i];
    const uint4 u = reinterpret_cast<const uint4*>(y)[i];
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const uint32_t a0 = apply_post_bits(bf16_bits_to_f32(gw[e] & 0xffffu), TPPX_POST_SILU, 0, 0, 1.0f);
      const uint32_t a1 = apply_post_bits(bf16_bits_to_f32(gw[e] >> 16), TPPX_POST_SILU, 0, 0, 1.0f);
      const uint32_t b0 = apply_post_bits(bf16_bits_to_f32(uw[e] & 0xffffu), TPPX_POST_MUL, a0, 0, 1.0f);
      const uint32_t b1 = apply_post_bits(bf16_bits_to_f32(uw[e] >> 16), TPPX_POST_MUL, a1, 0, 1.0f);
      o[e] = (b0 & 0xffffu) | (b1 << 16);
    }
    reinterpret_cast<uint4*>(y)[i] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

hipError_t launch_tiled_bf16(const TiledParams& p, hipStream_t stream) {
  // prompt-sized passes: the 128 x 256 form of the large MXFP4 kernel with the weights read as they are (two
  // workgroups of four waves per CU); its 32-bit offsets want operands below 4 GiB
  if (p.M >= big_min_rows() && env_int("TPPX_BF16_BIG", 1) != 0 &&
      (int64_t)p.M * p.K * 2 < ((int64_t)1 << 32) && (int64_t)p.tiles * 32 * p.K < ((int64_t)1 << 32)) {
    BigParams P;
    memset(&P, 0, sizeof(P));
    P.seg[0] = p;
    // (the 256 x 256 and 128 x 512 forms of eight waves were measured too: equal at 28672 x 8192, 20-30 % slower
    // at the 7B shapes)
    const int nb = (p.tiles + 15) / 16;
    for (int i = 1; i <= TPPX_MAX_SEGS; i++)
      P.nb0[i] = nb;
    P.n_seg = 1;
    P.xm = 1;
    // 64 x 128 workgroups, as for MXFP4, while there are at most 256 of them (with 2-byte weights they lose earlier:
    // 11008 x 4096 at 192 rows, 258 workgroups: 62 us against 52)
    if (((p.M + 63) / 64) * ((p.tiles + 7) / 8) <= 256 && env_int("TPPX_TILED_SMALL", 1) != 0) {
      const int nbs = (p.tiles + 7) / 8;
      for (int i = 1; i <= TPPX_MAX_SEGS; i++)
        P.nb0[i] = nbs;
      return big_bf16_launch<2, 2, 2>(P, ((p.M + 63) / 64) * nbs, stream);
    }
    if (((p.M + 127) / 128) * nb <= 256 && env_int("TPPX_TILED_W8", 1) != 0) // at most one workgroup per CU: eight waves, as for MXFP4
      return big_bf16_launch<4, 2, 4>(P, ((p.M + 127) / 128) * nb, stream);
    return big_bf16_launch<8, 1, 4>(P, ((p.M + 127) / 128) * nb, stream);
  }
  const int MB = (p.M + 127) / 128, NB = (p.tiles + 7) / 8;
  const dim3 grid((unsigned)(MB * NB));
  const size_t lds = 2 * 2048 * 16;
  TPPX_PLAN_ONLY(tiled_bf16_kernel, grid, dim3(256), lds);
  hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(tiled_bf16_kernel), lds);
  if (e != hipSuccess)
    return e;
  tiled_bf16_kernel<<<grid, 256, lds, stream>>>(p);
  return hipGetLastError();
}

hipError_t launch_silu_mul(const uint16_t* gate, uint16_t* y, int64_t n, hipStream_t stream) {
  const int64_t n8 = n / 8;
  const unsigned blocks = (unsigned)((n8 + 255) / 256 < 256 * 16 ? (n8 + 255) / 256 : 256 * 16);
  TPPX_PLAN_ONLY(silu_mul_kernel, dim3(blocks), dim3(256), 0);
  silu_mul_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(gate, y, n8);
  return hipGetLastError();
}

bool tiled_qint8_takes_groups(const TiledParams& p) {
  return p.qbs == 256 && p.M >= big_min_rows() && env_int("TPPX_TILED_BIG_QINT8", 1) != 0 &&
         (int64_t)p.M * p.K < ((int64_t)1 << 32) && (int64_t)p.tiles * 16 * p.K < ((int64_t)1 << 32);
}

// n GEMMs over the same quantised activations (same M, K, xq, sa) in one launch of the large-M kernel
hipError_t launch_tiled_qint8_group(const TiledParams* t, int n, hipStream_t stream) {
  {
    BigParams P;
    memset(&P, 0, sizeof(P));
    int nb = 0;
    for (int i = 0; i < n; i++) {
      P.seg[i] = t[i];
      P.nb0[i] = nb;
      nb += (t[i].tiles + 15) / 16;
    }
    for (int i = n; i <= TPPX_MAX_SEGS; i++)
      P.nb0[i] = nb;
    P.n_seg = n;
    const int MB4 = (t[0].M + 127) / 128, NB16 = nb;
    const size_t lds = 8 * 64 * EP_LD * sizeof(float); // epilogue staging; >= the A and B buffers + the scale slots
    static_assert(8 * 64 * EP_LD * sizeof(float) >= 2 * 128 * 256 + 64 * 1024 + 4 * 128 * sizeof(float), "LDS plan");
    // launches of at most 128 workgroups of 128 x 256: twice as many of 64 x 256, so that fewer CUs stay empty
    if (MB4 * NB16 <= 128 && env_int("TPPX_TILED_SMALL", 1) != 0) {
      const int MB2 = (t[0].M + 63) / 64;
      TPPX_PLAN_ONLY(big_qint8_small_kernel, dim3(MB2 * NB16), dim3(512), lds);
      if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(big_qint8_small_kernel), lds); e != hipSuccess)
        return e;
      big_qint8_small_kernel<<<dim3(MB2 * NB16), dim3(512), lds, stream>>>(P);
      return hipGetLastError();
    }
    TPPX_PLAN_ONLY(big_qint8_kernel, dim3(MB4 * NB16), dim3(512), lds);
    if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(big_qint8_kernel), lds); e != hipSuccess)
      return e;
    big_qint8_kernel<<<dim3(MB4 * NB16), dim3(512), lds, stream>>>(P);
    return hipGetLastError();
  }
}

hipError_t launch_tiled_qint8(const TiledParams& p, hipStream_t stream) {
  if (tiled_qint8_takes_groups(p))
    return launch_tiled_qint8_group(&p, 1, stream);
  const int MB = (p.M + 127) / 128, NB = (p.tiles + 7) / 8;
  const size_t lds = 2 * 1024 * 16 + 2 * 128 * sizeof(float);
  TPPX_PLAN_ONLY(tiled_qint8_kernel, dim3(MB * NB), dim3(256), lds);
  tiled_qint8_kernel<<<dim3(MB * NB), dim3(256), lds, stream>>>(p);
  return hipGetLastError();
}

} // namespace tppx
