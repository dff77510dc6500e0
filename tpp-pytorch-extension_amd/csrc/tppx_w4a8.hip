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
#include "tppx_launch.h"

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


// ---------------------------------------------------------------------------
// Many rows (prompt passes): the same arithmetic on the bf16 MFMA.  An int8 activation and a weight integer times
// its block's power of two are both exact in bf16, and the fp32 sum of the 32 products of one MX block is an
// integer below 2^19 times that power of two -- exact whatever order the MFMA adds in.  So one K = 32 bf16 MFMA
// with a zero accumulator input gives float(int32 block sum) * 2^(e - 127) without the convert, and the fold that
// remains is ONE fp32 multiply-add per output and block, f = fma(sum, sa[row][block], f) -- the reference's
// fma(float(sum), sa * 2^(e - 127), f) with the power of two moved to the other factor, the same bits.  f starts
// at the bias and the blocks are folded in ascending order, as the reference's loop does.
//   weights: tppx_prepack_mxfp4_int8_wide, bf16 tiles [N/16][K/128][4 b][64 lanes (g, n)][8]: lane (g, n) of MX block
//            b of K tile kt holds W[n][kt*128 + b*32 + g*8 .. +7] (integer * 2^(e - 127)), 2 bytes per weight;
//   rows:    quant_act_w4a8_wide_kernel, the int8 values as bf16 in the same operand order
//            [K/128][MT16][4 b][64 lanes (g, m)][8] and the scales (times 6/127) [K/128][MT16/4][4 b][16 m][4 mt],
//            MT16 row tiles padded to a multiple of 8 (rows past M repeat row M - 1; their outputs are not stored).
// The weights are the MFMA's first operand, so a result tile is [channel][row]: a lane holds four consecutive
// channels of ONE row -- its scale is one number per row tile and block (four row tiles in one 16-byte LDS read)
// and its outputs leave as 8-byte stores.
// ---------------------------------------------------------------------------
struct W4A8WideParams {
  const uint16_t* xa;
  const float* sa;
  const uint16_t* wn;
  const uint16_t* bias;
  const uint16_t* post_in;
  const uint16_t* post_in2;
  uint16_t* y;
  int M, N, K, MT16, tiles, post_op;
  float post_scale;
};

__global__ void __launch_bounds__(256)
quant_act_w4a8_wide_kernel(const uint16_t* __restrict__ x, int M, int K, int MT16, uint16_t* __restrict__ xa,
                           float* __restrict__ sa) {
  // one workgroup per (row tile of 16, K tile of 128); thread = (m = tid & 15, g = tid >> 4 & 3, b = tid >> 6)
  const int tid = threadIdx.x, m16 = tid & 15, g = (tid >> 4) & 3, b = tid >> 6;
  const int mt = blockIdx.x, kt = blockIdx.y;
  const int m = min(mt * 16 + m16, M - 1);
  const uint4 raw = *reinterpret_cast<const uint4*>(x + (int64_t)m * K + kt * 128 + b * 32 + g * 8);
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  float v[8];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    v[2 * i] = bf16_bits_to_f32(w[i] & 0xffffu);
    v[2 * i + 1] = bf16_bits_to_f32(w[i] >> 16);
    amax = fmaxf(amax, fmaxf(fabsf(v[2 * i]), fabsf(v[2 * i + 1])));
  }
  amax = fmaxf(amax, __shfl_xor(amax, 16, 64)); // the four lanes (g) of a (row, block)
  amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
  const float sc = __fdiv_rn(amax, 127.0f); // quantize_int8sym: scale = max / 127, q = rint(v * (1 / scale))
  const float inv = sc != 0.0f ? __frcp_rn(sc) : 0.0f;
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const float q0 = fminf(fmaxf(rintf(__fmul_rn(v[2 * i], inv)), -127.0f), 127.0f);
    const float q1 = fminf(fmaxf(rintf(__fmul_rn(v[2 * i + 1], inv)), -127.0f), 127.0f);
    o[i] = (__float_as_uint(q0) >> 16) | (__float_as_uint(q1) & 0xffff0000u); // integers up to 127 are exact in bf16
  }
  const int64_t slot = (((int64_t)kt * MT16 + mt) * 4 + b) * 64 + g * 16 + m16;
  reinterpret_cast<uint4*>(xa)[slot] = make_uint4(o[0], o[1], o[2], o[3]);
  if (g == 0)
    sa[((((int64_t)kt * (MT16 >> 2) + (mt >> 2)) * 4 + b) * 16 + m16) * 4 + (mt & 3)] = __fmul_rn(sc, (float)(6.0 / 127.0));
}

__global__ void __launch_bounds__(256)
prepack_w4a8_wide_kernel(const uint32_t* __restrict__ qref, const uint8_t* __restrict__ sref, int64_t N, int64_t K,
                         int64_t bc, uint4* __restrict__ wn) {
  // one thread per (channel tile, K tile, block b, lane (g, n)): eight weights of one channel
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t KT = K / 128;
  if (t >= (N / 16) * KT * 256)
    return;
  const int c = (int)(t & 15), g = (int)(t >> 4) & 3, b = (int)(t >> 6) & 3;
  const int64_t tile = t >> 8, kt = tile % KT, ntile = tile / KT;
  const int64_t n = ntile * 16 + c, n8b = n >> 3, n8 = n & 7;
  const int64_t C1 = K / bc, G = bc / 8, SB = bc / 32;
  const int64_t k0 = (kt * 4 + b) * 32, c1 = k0 / bc, kb = k0 % bc;
  const uint32_t codes = qref[((n8b * C1 + c1) * G + (kb >> 3) + g) * 8 + n8]; // byte i = value i | value 4 + i << 4
  const float ws = e8m0_to_f32(sref[((n8b * C1 + c1) * SB + (kb >> 5)) * 8 + n8]);
  const uint32_t lo = w4a8_expand(codes & 0x0F0F0F0Fu), hi = w4a8_expand((codes >> 4) & 0x0F0F0F0Fu);
  uint32_t h[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    h[i] = __float_as_uint(__fmul_rn((float)(int8_t)(lo >> (8 * i)), ws)) >> 16; // 7 bits times a power of two: exact
    h[4 + i] = __float_as_uint(__fmul_rn((float)(int8_t)(hi >> (8 * i)), ws)) >> 16;
  }
  wn[t] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
}

// A workgroup of four waves owns 128 rows x 128 channels (waves 2 x 2, a wave 64 x 64), two workgroups per CU, so
// that one computes while the other stands at its barrier.  K moves in tiles of 128 (four MX blocks): the rows
// (32 KiB) and their scales (2 KiB) are requested into registers a tile ahead and stored into the other of two LDS
// buffers at the end of the tile; the weights go from memory into a register ring, block b of the next tile
// requested behind the last MFMA that used block b of this one.  The kernel is bound by vector issue, not by the
// matrix pipe: 64 multiply-adds per lane and block beside 16 MFMAs.  (Tried and dropped: 256 x 128 workgroups of
// eight waves with every operand through LDS, by loads into registers or straight into LDS -- those take about
// 2.5 us to land on this part whatever they hit -- were 5-15 % slower: half the work per barrier.)
// MTW = row tiles of 16 per wave: 4 (workgroup 128 x 128) or 2 (64 x 128: twice as many workgroups for launches that
// would leave CUs empty or at one wave per SIMD).
template <int MTW>
__global__ void __launch_bounds__(256, 2)
linear_w4a8_wide_kernel(const W4A8WideParams p) {
  constexpr int WMT = MTW * 2; // row tiles per workgroup
  extern __shared__ __align__(16) uint8_t w4_lds[];
  // LDS: rows 2 buffers x [WMT mt][4 b][64 lanes] x 16 B (32 KiB each at most), then scales 2 buffers x
  // [groups of 64 rows][4 b][16 m] x 16 B
  i32x4* As = reinterpret_cast<i32x4*>(w4_lds);
  i32x4* Ss = reinterpret_cast<i32x4*>(w4_lds + 2 * 32768);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1, g = lane >> 4;
  const int MB = p.MT16 / WMT, NB = (p.tiles + 7) >> 3;
  int id = blockIdx.x;
  const int T = MB * NB;
  if ((T & 7) == 0) // workgroup ids go round the 8 XCDs: give each an eighth of the tiles, row blocks fastest
    id = (id & 7) * (T >> 3) + (id >> 3);
  const int bm = id % MB, bn = id / MB;
  const int KT = p.K >> 7;
  const int tile_base = bn * 8 + wn * 4;

  const i32x4* wq[4];
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int64_t t = min(tile_base + nt, p.tiles - 1);
    wq[nt] = reinterpret_cast<const i32x4*>(p.wn) + t * KT * 256 + lane;
  }
  const i32x4* xa = reinterpret_cast<const i32x4*>(p.xa) + (int64_t)bm * WMT * 256 + tid;
  const i32x4* sa = reinterpret_cast<const i32x4*>(p.sa) + (int64_t)bm * WMT * 16 + (tid & (WMT * 16 - 1));
  const int64_t xa_kt = (int64_t)p.MT16 * 256, sa_kt = (int64_t)p.MT16 * 16;

  i32x4 areg[WMT], sreg;
  i32x4 bring[4][4]; // [b][nt]
  auto load_a = [&](int ks) {
#pragma unroll
    for (int q = 0; q < WMT; q++)
      areg[q] = xa[ks * xa_kt + q * 256];
    sreg = sa[ks * sa_kt]; // WMT * 256 bytes of scales: the other waves fetch and store the same values again
  };
  auto load_b = [&](int ks, int b) {
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
      bring[b][nt] = wq[nt][(int64_t)ks * 256 + b * 64];
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int q = 0; q < WMT; q++)
      As[buf * 2048 + q * 256 + tid] = areg[q];
    Ss[buf * 128 + (tid & (WMT * 16 - 1))] = sreg;
  };

  f32x4 f[MTW][4]; // [mt][nt][r]: row mt*16 + (lane & 15), channel nt*16 + g*4 + r
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int n = min(tile_base + nt, p.tiles - 1) * 16 + g * 4;
    f32x4 bv = f32x4{0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
      const uint2 bb = *reinterpret_cast<const uint2*>(p.bias + n);
      bv = f32x4{bf16_bits_to_f32(bb.x & 0xffffu), bf16_bits_to_f32(bb.x >> 16), bf16_bits_to_f32(bb.y & 0xffffu),
                 bf16_bits_to_f32(bb.y >> 16)};
    }
#pragma unroll
    for (int mt = 0; mt < MTW; mt++)
      f[mt][nt] = bv;
  }

  load_a(0);
#pragma unroll
  for (int b = 0; b < 4; b++)
    load_b(0, b);
  store_a(0);
  __syncthreads();
  for (int ks = 0; ks < KT; ks++) {
    const int buf = ks & 1;
    // No branch in the K tile's body (the last tile requests itself again and nobody reads the copy): with branches
    // the compiler sinks every fold below the last one, behind all 64 MFMAs.
    const int kn = min(ks + 1, KT - 1);
    load_a(kn);
    const i32x4* Ab = As + buf * 2048 + (wm * MTW) * 256 + lane;
    // a group of 64 rows has its four row tiles' scales side by side: a wave of two row tiles reads its half of them
    const i32x4* Sb = Ss + buf * 128 + (MTW == 4 ? wm * 64 : 0) + (lane & 15);
    constexpr int NG = 4 * MTW; // groups (block b, row tile mt) of four MFMAs
    // NG groups of four MFMAs, fenced: left alone the compiler issues all 64 MFMAs of the K
    // tile first (none depends on another) and needs a register for every result.
    // The fold of a group runs under the MFMAs of the next one (results by the parity of the group).
    i32x4 sv[2];
    sv[0] = Sb[0];
    f32x4 t[2][4];
    static_for<0, NG + 1>([&](auto GI) {
      constexpr int gi = decltype(GI)::value;
      if constexpr (gi < NG) {
        constexpr int b = gi / MTW, mt = gi % MTW;
        const bf16x8 a = __builtin_bit_cast(bf16x8, Ab[mt * 256 + b * 64]);
        if constexpr (mt == 1 && b < 3) // (not at mt == 0: block b - 1's last fold, below, still reads that register)
          sv[(b + 1) & 1] = Sb[(b + 1) * 16];
        // weights first: the result tile is [channel][row], a lane holds four consecutive channels of one row
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
          t[gi & 1][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, bring[b][nt]), a,
                                                                  f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      }
      if constexpr (gi > 0) {
        constexpr int pb = (gi - 1) / MTW, pmt = (gi - 1) % MTW;
        const f32x4 sq = __builtin_bit_cast(f32x4, sv[pb & 1]);
        const float sc = MTW == 4 ? sq[pmt] : (wm ? sq[2 + pmt] : sq[pmt]);
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
          for (int r = 0; r < 4; r++)
            f[pmt][nt][r] = fmaf(t[(gi - 1) & 1][nt][r], sc, f[pmt][nt][r]);
        if constexpr (pmt == MTW - 1)
          load_b(kn, pb);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    store_a(buf ^ 1);
    __syncthreads();
  }

  const int m_base = bm * (WMT * 16) + wm * (MTW * 16) + (lane & 15);
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int tile = tile_base + nt;
    if (tile >= p.tiles)
      continue;
    const int n = tile * 16 + g * 4;
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) {
      const int m = m_base + mt * 16;
      if (m >= p.M)
        continue;
      const int64_t o = (int64_t)m * p.N + n;
      uint2 i1 = make_uint2(0u, 0u), i2 = make_uint2(0u, 0u);
      if (p.post_in)
        i1 = *reinterpret_cast<const uint2*>(p.post_in + o);
      if (p.post_in2)
        i2 = *reinterpret_cast<const uint2*>(p.post_in2 + o);
      const uint32_t h0 = apply_post_bits(f[mt][nt][0], p.post_op, i1.x & 0xffffu, i2.x & 0xffffu, p.post_scale);
      const uint32_t h1 = apply_post_bits(f[mt][nt][1], p.post_op, i1.x >> 16, i2.x >> 16, p.post_scale);
      const uint32_t h2 = apply_post_bits(f[mt][nt][2], p.post_op, i1.y & 0xffffu, i2.y & 0xffffu, p.post_scale);
      const uint32_t h3 = apply_post_bits(f[mt][nt][3], p.post_op, i1.y >> 16, i2.y >> 16, p.post_scale);
      *reinterpret_cast<uint2*>(p.y + o) = make_uint2((h0 & 0xffffu) | (h1 << 16), (h2 & 0xffffu) | (h3 << 16));
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

extern "C" int tppx_prepack_mxfp4_int8_wide(const void* q_ref, const void* sc_ref, int64_t N, int64_t K, int64_t bc,
                                            void* w_nat, tppx_stream_t stream) {
  const char* who = "tppx_prepack_mxfp4_int8_wide";
  TPPX_REQUIRE(q_ref && sc_ref && w_nat, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(w_nat) && ((uintptr_t)q_ref & 3) == 0, TPPX_EINVAL, "%s: pointer misaligned", who);
  TPPX_REQUIRE(N > 0 && N % 16 == 0 && K > 0 && K % 128 == 0 && bc >= 32 && bc % 32 == 0 && K % bc == 0, TPPX_ESHAPE,
               "%s: N=%ld must be a multiple of 16, K=%ld of 128 and of the block %ld (a multiple of 32)", who, (long)N,
               (long)K, (long)bc);
  const int64_t threads = (N / 16) * (K / 128) * 256;
  TPPX_REQUIRE((threads + 255) / 256 < ((int64_t)1 << 31), TPPX_ESHAPE, "%s: weight too large", who);
  prepack_w4a8_wide_kernel<<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
      (const uint32_t*)q_ref, (const uint8_t*)sc_ref, N, K, bc, (uint4*)w_nat);
  return check_hip(hipGetLastError(), who);
}

// bytes of workspace the wide kernel wants: the rows as bf16 + their scales, rows padded to a multiple of 128
static int64_t w4a8_wide_ws_bytes(int64_t M, int64_t K) {
  const int64_t mpad = (M + 127) / 128 * 128;
  return mpad * K * 2 + mpad * (K / 32) * 4;
}

extern "C" int tppx_linear_mxfp4_int8_wide(const void* x, const void* w_nat, const void* bias, const void* post_in,
                                           const void* post_in2, void* y, int64_t M, int64_t N, int64_t K, int post_op,
                                           float post_scale, void* ws, int64_t ws_bytes, tppx_stream_t stream) {
  const char* who = "tppx_linear_mxfp4_int8_wide";
  TPPX_REQUIRE(x && w_nat && y, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(x) && aligned16(w_nat), TPPX_EINVAL, "%s: activation / weight pointer not 16-byte aligned", who);
  TPPX_REQUIRE((((uintptr_t)y | (uintptr_t)bias | (uintptr_t)post_in | (uintptr_t)post_in2) & 7) == 0, TPPX_EINVAL,
               "%s: output, bias and post-op inputs must be 8-byte aligned", who);
  TPPX_REQUIRE(post_op >= TPPX_POST_NONE && post_op <= TPPX_POST_RELU, TPPX_EINVAL, "%s: unknown post-op id %d", who, post_op);
  TPPX_REQUIRE(M >= 0 && M < (1 << 24), TPPX_ESHAPE, "%s: M=%ld out of range", who, (long)M);
  TPPX_REQUIRE(N > 0 && N % 16 == 0 && N < (1 << 24), TPPX_ESHAPE, "%s: N=%ld must be a positive multiple of 16", who, (long)N);
  TPPX_REQUIRE(K > 0 && K % 128 == 0 && K < (1 << 24), TPPX_ESHAPE, "%s: K=%ld must be a positive multiple of 128", who, (long)K);
  if (M == 0)
    return TPPX_OK;
  const int64_t need = w4a8_wide_ws_bytes(M, K);
  TPPX_REQUIRE(ws && aligned16(ws) && ws_bytes >= need, TPPX_EINVAL,
               "%s: the workspace must hold %ld bytes (16-byte aligned) for the quantized rows, got %ld", who, (long)need,
               (long)ws_bytes);
  const int64_t mt16 = (M + 127) / 128 * 8, kt = K / 128;
  const int64_t mb = mt16 / 8, nb = (N / 16 + 7) / 8;
  TPPX_REQUIRE(kt <= 65535 && mb * nb < ((int64_t)1 << 31), TPPX_ESHAPE, "%s: problem too large", who);
  W4A8WideParams p;
  p.xa = (const uint16_t*)ws;
  p.sa = (const float*)((const uint8_t*)ws + mt16 * 16 * K * 2);
  p.wn = (const uint16_t*)w_nat;
  p.bias = (const uint16_t*)bias;
  p.post_in = (const uint16_t*)post_in;
  p.post_in2 = (const uint16_t*)post_in2;
  p.y = (uint16_t*)y;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.MT16 = (int)mt16;
  p.tiles = (int)(N / 16);
  p.post_op = post_op;
  p.post_scale = post_scale;
  quant_act_w4a8_wide_kernel<<<dim3((unsigned)mt16, (unsigned)kt), dim3(256), 0, (hipStream_t)stream>>>(
      (const uint16_t*)x, p.M, p.K, p.MT16, (uint16_t*)ws, (float*)((uint8_t*)ws + mt16 * 16 * K * 2));
  int rc = check_hip(hipGetLastError(), who);
  if (rc != TPPX_OK)
    return rc;
  const size_t lds = 2 * 32768 + 2 * 2048;
  // launches of at most 256 workgroups of 128 x 128 (at most one per CU: one wave per SIMD): 64 x 128 ones, twice as many
  if (mb * nb <= 256) {
    rc = check_hip(allow_dynamic_lds(reinterpret_cast<const void*>(linear_w4a8_wide_kernel<2>), lds), who);
    if (rc != TPPX_OK)
      return rc;
    linear_w4a8_wide_kernel<2><<<dim3((unsigned)(mb * 2 * nb)), dim3(256), lds, (hipStream_t)stream>>>(p);
    return check_hip(hipGetLastError(), who);
  }
  rc = check_hip(allow_dynamic_lds(reinterpret_cast<const void*>(linear_w4a8_wide_kernel<4>), lds), who);
  if (rc != TPPX_OK)
    return rc;
  linear_w4a8_wide_kernel<4><<<dim3((unsigned)(mb * nb)), dim3(256), lds, (hipStream_t)stream>>>(p);
  return check_hip(hipGetLastError(), who);
}
