// Host-side launch descriptors shared by the C-ABI layer and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TPPX_MAX_SEGS 4

namespace tppx {

// One GEMM of a (possibly fused) group; device pointers.
struct SkinnySeg {
  const void* qw;           // native weight tiles
  const void* sw;           // scales (u8 native for MXFP4, f32 reference for QINT8)
  const uint16_t* bias;     // bf16 [N] or null
  const uint16_t* post_in;  // bf16 [M][N] or null
  const uint16_t* post_in2; // bf16 [M][N] or null
  uint16_t* y;              // bf16 [M][N]
  int N;
  int tile0;                // first 16-channel tile of this GEMM in the fused tile space
  int post_op;
  float post_scale;
};

struct SkinnyParams {
  SkinnySeg seg[TPPX_MAX_SEGS];
  int n_seg;
  const void* x;   // bf16 [M][K]            (MXFP4)
  const void* xq;  // int8 [M][K]            (QINT8)
  const float* sa; // f32  [M][K/qbs]        (QINT8)
  int M, K;
  int kunits;         // K/128 (MXFP4) or K/qbs (QINT8)
  int units_per_wave; // contiguous K units handled by one wave
  int qbs;
};

struct SkinnyPlan {
  int mg, nt, waves, units_per_wave, grid_x, grid_y;
};

int env_int(const char* name, int dflt);

SkinnyPlan plan_skinny(int64_t M, int total_tiles, int kunits, bool all_even, bool dual);
hipError_t launch_skinny_mxfp4(const SkinnyParams& p, const SkinnyPlan& pl, bool dual, hipStream_t stream);
hipError_t launch_skinny_qint8(const SkinnyParams& p, const SkinnyPlan& pl, hipStream_t stream);

} // namespace tppx
