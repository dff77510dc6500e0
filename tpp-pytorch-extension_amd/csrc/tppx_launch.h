// Host-side launch descriptors shared by the C-ABI layer and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#define TPPX_MAX_SEGS 4

namespace tppx {

// One GEMM of a (possibly fused) group; device pointers.
struct DecodeSeg {
  const void* qw;           // native weight tiles
  const void* sw;           // scales (u8 native for MXFP4, f32 reference for QINT8)
  const uint16_t* bias;     // bf16 [N] or null
  const uint16_t* post_in;  // bf16 [M][N] or null
  const uint16_t* post_in2; // bf16 [M][N] or null
  uint16_t* y;              // bf16 [M][N]
  int N;
  int tiles;                // N / 16
  int tile0;                // first tile of this GEMM in the fused tile space
  int grp0;                 // first workgroup (group of channel tiles) of this GEMM in the launch
  int post_op;
  float post_scale;
  // split1 > 0: the N output channels go to up to three row-major matrices laid one after the other in y
  // (columns [0, split1) | [split1, split2) | [split2, N): M x split1, then M x (split2 - split1), then the rest):
  // one GEMM over concatenated weights whose results are separate tensors (q, k, v)
  int split1, split2;
};

// element offset of output (m, n) of a segment in y (and in post_in / post_in2, which share its layout)
__host__ __device__ inline int seg_out_offset(const DecodeSeg& sg, int M, int m, int n) {
  if (sg.split1 <= 0)
    return m * sg.N + n;
  const int w0 = sg.split1, w1 = sg.split2 - sg.split1, w2 = sg.N - sg.split2;
  return n < sg.split1 ? m * w0 + n : n < sg.split2 ? M * w0 + m * w1 + (n - sg.split1) : M * (w0 + w1) + m * w2 + (n - sg.split2);
}

struct DecodeParams {
  DecodeSeg seg[TPPX_MAX_SEGS];
  int n_seg;
  int groups;      // workgroups along x: sum over segments of ceil(tiles / tiles per workgroup)
  int total_tiles; // sum of tiles (one segment's tiles for the dual gate/up kernel)
  const void* x;   // bf16 [M][K]
  const void* xq;  // int8 [M][K], or MFMA operand order when mt > 0 (QINT8, unless quantised in-kernel)
  const float* sa; // f32  [M][K/qbs] (QINT8, unless quantised in-kernel)
  int M, K;
  int mt;    // > 0: xq is [K/64][mt][4 g][16 m][16 B] (operand tiles of 16 rows x 64 K); 0: row-major
  int units; // what is dealt to waves (and K parts): K/128 (MXFP4 tiles); QINT8: K / (64 * deal)
  int tpb;   // native tiles per scale block (1 for MXFP4, qbs/64 for QINT8)
  // QINT8: K is dealt in runs of `deal` 64-wide tiles: 4 (256 input channels) when a scale block is a whole number of
  // such runs, whole blocks when a block has fewer than 4 tiles, single tiles otherwise.  A run that ends inside a
  // scale block folds its exact int32 sums with the block's scales like a block of its own.
  int deal;
  int nblk;  // QINT8: K / qbs scale blocks
  int wbits; // QINT8 family, fused-quantisation kernel: 4 or 2 = seg[].qw holds packed codes (tppx_pack_qint_tiles); else int8 tiles
  // deal == 4: scale block of run u = spb_magic ? mulhi(u, spb_magic) : u   (spb_magic = ceil(2^32 / (tpb / 4)),
  // exact for u * (tpb / 4) < 2^32; 0 when a block is one run)
  unsigned int spb_magic;
  // fused-quantisation kernel: (row, run) item i -> run i / M as mulhi(i, m_magic), m_magic = ceil(2^32 / M) (exact
  // for i < 2^17, M <= 16); 0 when M == 1
  unsigned int m_magic;
  // 17..64-row kernel: scale block of tile t = tpb_magic ? mulhi(t, tpb_magic) : t   (ceil(2^32 / tpb); 0 when tpb == 1)
  unsigned int tpb_magic;
  int S;     // K parts across workgroups (grid z, at most 4); > 1: partial sums go to `part`, the workgroup that
             // arrives last at its ticket adds them and runs the epilogue
  int ticket0; // first arrival counter of this launch (S > 1), see skinny_split_tickets()
  int cht;   // tiles of activations staged in LDS at a time
  int lds_overlap; // fused-quantisation QINT8 kernel: the reduction region reuses the LDS of the activations
  float* part;   // [S][block row][total_tiles][MG][256] fp32 partial tiles (S > 1)
  const float* norm_gamma; // f32 [K]: RMSNorm fused in front of the GEMM (LDS-staged MXFP4 kernel), or null
  float norm_eps;
  // Row sums of squares handed from the GEMM that writes a tensor to the GEMM that normalises it: f32 [16][256],
  // entry [row][workgroup] = sum of squares of the bf16 outputs of that row owned by that workgroup (unused
  // workgroup slots zero).  The consumer adds a row's 256 entries instead of making a pass over the row.
  float* sumsq_out;      // written by this launch's epilogue (M <= 16, single GEMM), or null
  const float* sumsq_in; // with norm_gamma: the table the launch that produced x wrote, or null (sum x^2 here)
};

// launch shape of the QINT8 decode kernels (K split inside the workgroup)
struct SkinnyPlan {
  int mg, ntw, waves, max_units, grid_y;
  bool fused_quant; // QINT8, M <= 16: activations quantised inside the GEMM kernel
  bool lds_overlap; // ... and its reduction region reuses the LDS of the quantised activations
};

// one GEMM on the LDS-tiled (prefill) kernels
struct TiledParams {
  const void* x;   // bf16 [M][K]           (MXFP4)
  const void* xq;  // int8 [M][K]           (QINT8)
  const float* sa; // f32  [M][K/qbs]       (QINT8)
  const void* qw;
  const void* sw;
  const uint16_t* bias;
  const uint16_t* post_in;
  const uint16_t* post_in2;
  uint16_t* y;
  int M, N, K;
  int tiles; // N / 16
  int qbs;
  int post_op;
  float post_scale;
};

hipError_t launch_tiled_mxfp4(const TiledParams& p, hipStream_t stream);
// large-M kernel: several GEMMs over one activation in one launch
bool tiled_mxfp4_takes_groups(const TiledParams& p);
// dual: the gate/up pair (t[0] = gate, t[1] = up) with silu(gate) * up formed in the launch and written to t[1].y
hipError_t launch_tiled_mxfp4_group(const TiledParams* t, int n, hipStream_t stream, bool dual = false);
hipError_t launch_tiled_qint8(const TiledParams& p, hipStream_t stream);
// unquantized bf16 weights (native bf16 tiles in p.qw), more than 64 rows
hipError_t launch_tiled_bf16(const TiledParams& p, hipStream_t stream);
hipError_t launch_tiled_mxfp4_fp8_group(const TiledParams* t, int n, hipStream_t stream, bool dual = false);
bool tiled_qint8_takes_groups(const TiledParams& p);
hipError_t launch_tiled_qint8_group(const TiledParams* t, int n, hipStream_t stream);
// y[i] = bf16( silu(gate[i]) * y[i] ) with the rounding points of SiluPostOp followed by MulPostOp; n % 8 == 0
hipError_t launch_silu_mul(const uint16_t* gate, uint16_t* y, int64_t n, hipStream_t stream);

int env_int(const char* name, int dflt);
// rows from which the prefill kernels of 128-row workgroups (and their 64-row forms for small launches) take a
// GEMM; below it the older 128 x 128 kernels run.  (It was 192 before the 64-row forms existed: at 4096 x 4096 and
// 160 rows they take 26 us where the old kernels took 62-88; TPPX_TILED_BIG_MIN_M overrides.)
inline int big_min_rows() { return env_int("TPPX_TILED_BIG_MIN_M", 65); }
// dynamic LDS above 48 KiB must be allowed per kernel and device before the launch
hipError_t allow_dynamic_lds(const void* kern, size_t lds);

// dynamic activation quantisation; mt > 0 writes xq in MFMA operand order (see DecodeParams::mt)
hipError_t launch_quant_act_int8(const void* x, int64_t M, int64_t K, int64_t qbs, void* xq, void* sa, int mt,
                                 hipStream_t stream);

// MXFP8 activations in MFMA operand order for the block-scaled prefill kernel: rows padded to Mp = roundup(M, 64);
// xq Mp*K bytes, xs Mp*K/32 bytes
hipError_t launch_quant_act_mxfp8(const void* x, int64_t M, int64_t K, void* xq, void* xs, hipStream_t stream);

// units = runs of K dealt to waves (DecodeParams::units), tpb / deal as in DecodeParams;
// can_fuse_quant: bf16 activations at hand and blocks of a multiple of 256 (the in-kernel quantisation's case)
SkinnyPlan plan_skinny(int64_t M, int total_tiles, int units, int tpb, int deal, bool can_fuse_quant);
// scale blocks a wave that owns `runs` consecutive runs of K can touch
int skinny_qint8_blocks_per_wave(int runs, int tpb, int deal, int nblk);
hipError_t launch_skinny_qint8(DecodeParams& p, const SkinnyPlan& pl, hipStream_t stream);
hipError_t launch_skinny_qint8_nk(DecodeParams& p, int mg, hipStream_t stream);
// QINT4 / QINT2 codes at their own width, 17..64 rows per block row: mg = 2 / 4 row groups, ntw = 1..3 channel tiles
// per workgroup; p.wbits, p.mt (operand-order activations) and p.groups set by the caller
hipError_t launch_skinny_qintx(DecodeParams& p, int mg, int ntw, hipStream_t stream);
// W4A8 decode kernel (M <= 16): does it fit (LDS), and with how many channel tiles per workgroup; p.units = K / 128
bool skinny_w4a8_fits(int64_t M, int total_tiles, int ktiles, int* ntw_out);
hipError_t launch_skinny_w4a8(DecodeParams& p, int ntw, hipStream_t stream);
hipError_t launch_skinny_mxfp4_nk(DecodeParams& p, hipStream_t stream);
hipError_t launch_skinny_bf16(DecodeParams& p, int mg, int nt, hipStream_t stream);
size_t skinny_mxfp4_xl_lds(int units, int nt, bool dual);
hipError_t launch_skinny_mxfp4_x4(DecodeParams& p, int nt, bool dual, hipStream_t stream);
hipError_t launch_skinny_mxfp4_mg(DecodeParams& p, int mg, int nt, bool dual, hipStream_t stream);
hipError_t launch_skinny_mxfp4_xl(DecodeParams& p, int nt, bool dual, hipStream_t stream);

// window of `n` arrival counters for one K-split launch (first index), or -1 when n exceeds what the library keeps
int skinny_split_tickets(int n);

} // namespace tppx
