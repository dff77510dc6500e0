// Second pass of the decode kernels that split K across workgroups.
//
// Those kernels leave their sums in the caller's workspace as accumulator
// fragments, [K part][block row][tile][row group][lane] x f32x4 (lane l, value
// r = row (l >> 4) * 4 + r, channel l & 15 of the 16 x 16 tile).  One wave per
// (tile, row group) adds the parts in a fixed order and runs the fused
// epilogue (bias -> bf16 -> post-op -> bf16).
#include "tppx_common.h"
#include "tppx_launch.h"

namespace tppx {

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
  const int gy = (p.M + MG * 16 - 1) / (MG * 16); // block rows of the first pass
  if (wid >= per_y * gy)
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
  const int64_t ks_stride = (int64_t)gy * p.total_tiles * NACC * MG * 64;
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

hipError_t launch_splitk_finish(const DecodeParams& p, int mg, int grid_y, hipStream_t stream) {
  const int64_t waves = (int64_t)p.total_tiles * mg * grid_y;
  const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
#define FIN(MG)                                                     \
  {                                                                 \
    TPPX_PLAN_ONLY((splitk_finish_kernel<MG, false>), grid, block, 0); \
    splitk_finish_kernel<MG, false><<<grid, block, 0, stream>>>(p); \
    return hipGetLastError();                                       \
  }
  switch (mg) {
    case 1: FIN(1)
    case 2: FIN(2)
    default: FIN(4)
  }
#undef FIN
}

} // namespace tppx
