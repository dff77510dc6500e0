// Decode-side operators around the quantized linears of a Llama decoder layer:
// RMSNorm, rotary position embedding, KV-cache append and single-query
// (decode) attention.  All of them are bandwidth bound: one pass over their
// inputs with 128-bit coalesced accesses, reductions inside a wave with DPP,
// fp32 arithmetic, one bf16 rounding where the CPU path stores bf16.
#include <math.h>
#include <string.h>

#include <mutex>

#include "tppx_common.h"
#include "tppx_launch.h"

namespace tppx {

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// sum / max over the 16 lanes of a DPP row; every lane of the row gets the result
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_mov<0xB1>(v);  // quad_perm [1,0,3,2]
  v += dpp_mov<0x4E>(v);  // quad_perm [2,3,0,1]
  v += dpp_mov<0x141>(v); // row_half_mirror
  v += dpp_mov<0x140>(v); // row_mirror
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (a + b) + (c + d);
}

__device__ __forceinline__ void unpack8(const uint4& w, float (&f)[8]) {
  const uint32_t d[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    f[2 * i] = bf16_bits_to_f32(d[i] & 0xffffu);
    f[2 * i + 1] = bf16_bits_to_f32(d[i] >> 16);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  uint32_t d[4];
#pragma unroll
  for (int i = 0; i < 4; i++)
    d[i] = f32_to_bf16_bits(f[2 * i]) | (f32_to_bf16_bits(f[2 * i + 1]) << 16);
  return make_uint4(d[0], d[1], d[2], d[3]);
}

// ---------------------------------------------------------------------------
// RMSNorm: y = bf16( (x * rsqrt(mean(x^2) + eps)) * gamma ), fp32 inside.
// One workgroup of 256 threads per row; K a multiple of 8.
// ---------------------------------------------------------------------------
template <bool GAMMA_F32>
__global__ void __launch_bounds__(256)
rms_norm_kernel(const uint16_t* __restrict__ x, const void* __restrict__ gamma, uint16_t* __restrict__ y,
                int K, float eps) {
  __shared__ float red[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const uint4* xr = reinterpret_cast<const uint4*>(x + (int64_t)row * K);
  uint4* yr = reinterpret_cast<uint4*>(y + (int64_t)row * K);
  const int nchunk = K >> 3;
  float ss = 0.f;
  for (int i = tid; i < nchunk; i += 256) {
    float f[8];
    unpack8(xr[i], f);
#pragma unroll
    for (int e = 0; e < 8; e++)
      ss = fmaf(f[e], f[e], ss);
  }
  ss = wave_sum(ss);
  if ((tid & 63) == 0)
    red[tid >> 6] = ss;
  __syncthreads();
  const float v = ((red[0] + red[1]) + (red[2] + red[3])) * (1.0f / (float)K);
  const float s = 1.0f / sqrtf(v + eps);
  for (int i = tid; i < nchunk; i += 256) {
    float f[8], g[8];
    unpack8(xr[i], f); // second read hits L2/L1
    if (GAMMA_F32) {
      const float4* gp = reinterpret_cast<const float4*>(gamma) + 2 * i;
      const float4 g0 = gp[0], g1 = gp[1];
      g[0] = g0.x; g[1] = g0.y; g[2] = g0.z; g[3] = g0.w;
      g[4] = g1.x; g[5] = g1.y; g[6] = g1.z; g[7] = g1.w;
    } else {
      unpack8(reinterpret_cast<const uint4*>(gamma)[i], g);
    }
#pragma unroll
    for (int e = 0; e < 8; e++)
      f[e] = (f[e] * s) * g[e];
    yr[i] = pack8(f);
  }
}

// ---------------------------------------------------------------------------
// LayerNorm (lyr_norm, fused_llm_infer.cpp:254-306; LayerNormFwdTPP,
// xsmm_functors.h:4749-4786): m = mean(x), v = max(mean(x^2) - m^2, 0),
// s = 1 / sqrt(v + eps), y = bf16( (x * s - s * m) * gamma + beta ), fp32 inside.
// One workgroup of 256 threads per row; K a multiple of 8.
// ---------------------------------------------------------------------------
template <bool PARAMS_F32>
__device__ __forceinline__ void load8_param(const void* p, int i, float (&g)[8]) {
  if (PARAMS_F32) {
    const float4* gp = reinterpret_cast<const float4*>(p) + 2 * i;
    const float4 g0 = gp[0], g1 = gp[1];
    g[0] = g0.x; g[1] = g0.y; g[2] = g0.z; g[3] = g0.w;
    g[4] = g1.x; g[5] = g1.y; g[6] = g1.z; g[7] = g1.w;
  } else {
    unpack8(reinterpret_cast<const uint4*>(p)[i], g);
  }
}

template <bool PARAMS_F32>
__global__ void __launch_bounds__(256)
layer_norm_kernel(const uint16_t* __restrict__ x, const void* __restrict__ gamma, const void* __restrict__ beta,
                  uint16_t* __restrict__ y, int K, float eps) {
  __shared__ float red[2][4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const uint4* xr = reinterpret_cast<const uint4*>(x + (int64_t)row * K);
  uint4* yr = reinterpret_cast<uint4*>(y + (int64_t)row * K);
  const int nchunk = K >> 3;
  float sm = 0.f, ss = 0.f;
  for (int i = tid; i < nchunk; i += 256) {
    float f[8];
    unpack8(xr[i], f);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      sm += f[e];
      ss = fmaf(f[e], f[e], ss);
    }
  }
  sm = wave_sum(sm);
  ss = wave_sum(ss);
  if ((tid & 63) == 0) {
    red[0][tid >> 6] = sm;
    red[1][tid >> 6] = ss;
  }
  __syncthreads();
  const float c = 1.0f / (float)K;
  const float m = ((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) * c;
  float v = ((red[1][0] + red[1][1]) + (red[1][2] + red[1][3])) * c;
  v = fmaxf(v - m * m, 0.0f);
  const float s = 1.0f / sqrtf(v + eps);
  const float b = -1.0f * s * m;
  for (int i = tid; i < nchunk; i += 256) {
    float f[8], g[8], bt[8];
    unpack8(xr[i], f); // second read hits L2/L1
    load8_param<PARAMS_F32>(gamma, i, g);
    load8_param<PARAMS_F32>(beta, i, bt);
#pragma unroll
    for (int e = 0; e < 8; e++)
      f[e] = (f[e] * s + b) * g[e] + bt[e];
    yr[i] = pack8(f);
  }
}

// ---------------------------------------------------------------------------
// Llama rotary embedding, in place on t [B][S][N][H] (rotate-half pairs
// (h2, HR/2 + h2)), cos/sin table f32 [2][MP][HR], positions i64 [B_pos][S].
// Optionally the rotated key rows and the value rows are also written into
// the KV cache [B][N][Smax][H] at position offset + s (offset read from device
// memory), so that one launch covers rotary(q), rotary(k) and the cache append.
// One thread per (token, head, pair of 8-wide chunks).
// ---------------------------------------------------------------------------
struct RotaryParams {
  uint16_t* q;         // [B][S][Nq][H] or null
  uint16_t* k;         // [B][S][Nkv][H] or null
  const uint16_t* v;   // [B][S][Nkv][H] or null (append only)
  uint16_t* kc;        // [B][Nkv][Smax][H] or null
  uint16_t* vc;
  const float* emb;    // [2][MP][HR] or null (append without rotation)
  const int64_t* pos;  // [B_pos][S]
  const int32_t* offset; // device scalar: cache length before this append
  int B, S, Nq, Nkv, H, MP, HR, B_pos, Smax;
  int gptj;            // 1: GPT-J pairs (h, h + 1) and a sin | cos table f32 [MP][HR] (fused_llm_infer.cpp:150-205)
};

__global__ void __launch_bounds__(256)
rotary_append_kernel(const RotaryParams p) {
  // work item = (b, s, head in [0, Nq + Nkv + Nkv), chunk c of H/8); the pair partner is fetched by the same thread
  const int CH = p.H >> 3;
  const int heads = (p.q ? p.Nq : 0) + (p.k ? p.Nkv : 0) + ((p.v && p.vc) ? p.Nkv : 0);
  const int64_t total = (int64_t)p.B * p.S * heads * CH;
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total)
    return;
  const int c = (int)(id % CH);
  int hh = (int)((id / CH) % heads);
  const int64_t tok = id / ((int64_t)CH * heads);
  const int s = (int)(tok % p.S), b = (int)(tok / p.S);
  const int nq = p.q ? p.Nq : 0, nk = p.k ? p.Nkv : 0;
  const int off = (p.kc || p.vc) ? *p.offset : 0;
  if (hh >= nq + nk) { // value rows: plain copy into the cache
    const int n = hh - nq - nk;
    const uint4 w = reinterpret_cast<const uint4*>(p.v + (((int64_t)b * p.S + s) * p.Nkv + n) * p.H)[c];
    if (off + s < p.Smax)
      reinterpret_cast<uint4*>(p.vc + (((int64_t)b * p.Nkv + n) * p.Smax + off + s) * p.H)[c] = w;
    return;
  }
  const bool is_k = hh >= nq;
  const int n = is_k ? hh - nq : hh;
  uint16_t* row = is_k ? p.k + (((int64_t)b * p.S + s) * p.Nkv + n) * p.H
                       : p.q + (((int64_t)b * p.S + s) * p.Nq + n) * p.H;
  uint4 w = reinterpret_cast<uint4*>(row)[c];
  const int coff = p.HR >> 1;
  const int h0 = c * 8;
  const int64_t pp = p.pos[(int64_t)(p.B_pos == 1 ? 0 : b) * p.S + s];
  if (p.gptj) {
    if (p.emb && h0 < p.HR && pp >= 0 && pp < p.MP) {
      // a chunk of 8 holds four whole pairs (h, h + 1); sin at [p][h / 2], cos at [p][HR / 2 + h / 2]
      float a[8], r[8];
      unpack8(w, a);
      const float* sn = p.emb + pp * p.HR + (h0 >> 1);
      const float* cs = sn + coff;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        r[2 * e] = a[2 * e] * cs[e] - a[2 * e + 1] * sn[e];
        r[2 * e + 1] = a[2 * e + 1] * cs[e] + a[2 * e] * sn[e];
      }
      w = pack8(r);
    }
  } else if (p.emb && h0 < p.HR && pp >= 0 && pp < p.MP) { // positions outside the table are left unrotated
    // this chunk holds first halves (h0 < HR/2) or second halves of rotation pairs
    const bool first = h0 < coff;
    const int h2 = first ? h0 : h0 - coff;
    const int cp = first ? c + (coff >> 3) : c - (coff >> 3); // the partner chunk
    const uint4 wo = reinterpret_cast<const uint4*>(row)[cp];
    float a[8], o[8], r[8];
    unpack8(w, a);
    unpack8(wo, o);
    const float* cs = p.emb + pp * p.HR + h2;
    const float* sn = p.emb + ((int64_t)p.MP + pp) * p.HR + h2;
    if ((CH & (CH - 1)) != 0) {
      // A head of a number of chunks that is no power of two can straddle two waves, and the partner thread in the
      // other wave might read this chunk after it has been rewritten: the thread of the first half writes both
      // chunks here, the thread of the second half writes nothing.
      if (!first)
        return;
      float r2[8];
#pragma unroll
      for (int e = 0; e < 8; e++) {
        r[e] = a[e] * cs[e] - o[e] * sn[e];
        r2[e] = o[e] * cs[e] + a[e] * sn[e];
      }
      const uint4 w2 = pack8(r2);
      reinterpret_cast<uint4*>(row)[cp] = w2;
      if (is_k && p.kc && off + s < p.Smax)
        reinterpret_cast<uint4*>(p.kc + (((int64_t)b * p.Nkv + n) * p.Smax + off + s) * p.H)[cp] = w2;
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) {
        // first half: in0*cos - in1*sin ; second half: in1*cos + in0*sin
        r[e] = first ? a[e] * cs[e] - o[e] * sn[e] : a[e] * cs[e] + o[e] * sn[e];
      }
    }
    w = pack8(r);
  }
  // The two threads of a rotation pair sit in the same wave (H/8 is a power of
  // two <= 64 and work items are numbered chunk-fastest), and this store needs
  // both loaded chunks, so the wave's loads have returned before it issues.
  reinterpret_cast<uint4*>(row)[c] = w;
  if (is_k && p.kc && off + s < p.Smax)
    reinterpret_cast<uint4*>(p.kc + (((int64_t)b * p.Nkv + n) * p.Smax + off + s) * p.H)[c] = w;
}

// ---------------------------------------------------------------------------
// Decode attention (one query token per sequence), head size 128, cache
// [B][Nkv][Smax][128] bf16.  Grid (B*Nq, splits); split y takes the trips
// y, y + splits, ... of the key range, whose length is a device scalar.  Two
// kernels share the split merge (attn_finish):
//   attn_decode_kernel       4 waves, a wave instruction reads 4 keys (lane =
//     key l>>4, 16-byte chunk l&15), 64 keys per trip with the next trip
//     requested ahead; every 16-lane row keeps its own running (max, sum, 8
//     output dims per lane), merged at the end through LDS: the long loops of
//     larger batches;
//   attn_decode_wide_kernel  128 keys per trip on the packed bf16 dot
//     instruction: the one- or two-trip workgroups of small batches, where
//     the arithmetic above costs more than the cache stream.
// Scores: fp32 dot * 1/sqrt(H) + mask; probabilities are rounded to bf16
// before they multiply V (as the CPU path stores them), sums and the output
// accumulate in fp32.
// ---------------------------------------------------------------------------
struct AttnParams {
  const uint16_t* q;    // [B][Nq][128]
  const uint16_t* kc;   // [B][Nkv][Smax][128]
  const uint16_t* vc;
  const uint16_t* mask; // bf16 [B][mask_ld] additive, or null
  const int32_t* kv_len; // device scalar; valid keys = *kv_len + kv_len_add
  int kv_len_add;
  uint16_t* out;        // [B][Nq][128]
  float* part;          // [B*Nq][splits][130]
  int B, Nq, Nkv, Smax, mask_ld, splits;
  int ticket0;          // >= 0: first arrival counter of this launch (the last split to arrive merges); < 0: second kernel
  float scale;
  // ROT: the query and the step's new key / value arrive unrotated and not yet in the cache
  const uint16_t* k_new; // [B][Nkv][128]
  const uint16_t* v_new; // [B][Nkv][128]
  const float* emb;      // f32 [2][MP][128] cos / sin
  const int64_t* pos;    // i64 [B_pos] position of the new token
  int MP, B_pos;
};

// Arrival counters of the split launches, one per (sequence, head): zero between launches (the counting
// instruction wraps on the last arrival); a launch takes a window handed out in rotation by the host.
// The counters of a launch are all hit within a microsecond or two; side by side they would queue up at the atomic
// unit of one memory channel, so each one has 256 bytes to itself.
constexpr int ATTN_TICKETS = 4096;
constexpr int ATTN_TICKET_STRIDE = 64; // in counters
__device__ unsigned int attn_tickets[ATTN_TICKETS * ATTN_TICKET_STRIDE];

__global__ void attn_clear_tickets_kernel(int first, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    attn_tickets[(first + i) * ATTN_TICKET_STRIDE] = 0;
}

__device__ __forceinline__ uint4 as_uint4(const i32x4& v) {
  return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}

// Shared end of the single-query kernels.  Threads tid < 128 hold output dimension tid of this workgroup's state: the
// running max M, the sum Ls and the unnormalised output o.  One split: normalise and store.  Several: store the state;
// with arrival counters the split that arrives last merges all of them inside the launch.
__device__ __forceinline__ void attn_finish(const AttnParams& p, int bh, int tid, float M, float Ls, float o) {
  if (tid < 128) {
    if (p.splits == 1) {
      p.out[(int64_t)bh * 128 + tid] = (uint16_t)f32_to_bf16_bits(Ls > 0.f ? o / Ls : 0.f);
    } else if (p.ticket0 < 0) {
      float* dst = p.part + ((int64_t)bh * p.splits + blockIdx.y) * 130;
      dst[2 + tid] = o;
      if (tid == 0) {
        dst[0] = M;
        dst[1] = Ls;
      }
    } else {
      // device-scope atomic stores: written through to the level all XCDs share, no cache write-back needed
      float* dst = p.part + ((int64_t)bh * p.splits + blockIdx.y) * 130;
      __hip_atomic_store(dst + 2 + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (tid == 0) {
        __hip_atomic_store(dst, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(dst + 1, Ls, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  if (p.splits == 1 || p.ticket0 < 0)
    return;
  // The split that arrives last merges all of them, in split order (the same sums whichever split that is).
  // Order: every thread waits until its own stores above have been acknowledged (vmcnt counts stores on this
  // target; a workgroup barrier by itself does not wait for the global stores of the other waves), then the
  // barrier, then the ticket, then the device-scope loads of the other splits' results.  Nobody waits for anybody.
  __shared__ int arrived_last;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    const unsigned int last = (unsigned int)p.splits - 1;
    arrived_last = atomicInc(&attn_tickets[(p.ticket0 + bh) * ATTN_TICKET_STRIDE], last) == last;
  }
  __syncthreads();
  if (!arrived_last || tid >= 128)
    return;
  const float* src = p.part + (int64_t)bh * p.splits * 130;
  float pm[32], pl[32], po[32]; // every load in flight at once (at most 32 splits)
#pragma unroll
  for (int i = 0; i < 32; i++) {
    pm[i] = -3.0e38f;
    pl[i] = po[i] = 0.f;
    if (i < p.splits) {
      pm[i] = __hip_atomic_load(src + i * 130, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      pl[i] = __hip_atomic_load(src + i * 130 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      po[i] = __hip_atomic_load(src + i * 130 + 2 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  M = -3.0e38f;
#pragma unroll
  for (int i = 0; i < 32; i++)
    if (i < p.splits)
      M = fmaxf(M, pm[i]);
  Ls = 0.f;
  o = 0.f;
#pragma unroll
  for (int i = 0; i < 32; i++)
    if (i < p.splits) {
      const float w = __expf(pm[i] - M);
      Ls = fmaf(w, pl[i], Ls);
      o = fmaf(w, po[i], o);
    }
  p.out[(int64_t)bh * 128 + tid] = (uint16_t)f32_to_bf16_bits(Ls > 0.f ? o / Ls : 0.f);
}


// ROT: the launch also does what the rotary + append launch did before it (fused_llm_infer.cpp:1252-1253 and
// LayerCache::update, attn.h:198-222): q and the new key arrive unrotated, every workgroup rotates its query, the
// key / value of the new token (cache position *kv_len) are taken from registers wherever that position is read,
// and one workgroup per KV head writes them into the cache.  Rotated values are rounded to bf16 first, as stored.
template <bool ROT>
__global__ void __launch_bounds__(256)
attn_decode_kernel(const AttnParams p) {
  __shared__ float sm[16], sl[16];
  __shared__ float sacc[16][128];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, c = lane & 15;
  const int bh = blockIdx.x, b = bh / p.Nq, hq = bh - b * p.Nq;
  const int hk = hq / (p.Nq / p.Nkv);
  const uint4* kb = reinterpret_cast<const uint4*>(p.kc + ((int64_t)b * p.Nkv + hk) * p.Smax * 128) + c;
  const uint4* vb = reinterpret_cast<const uint4*>(p.vc + ((int64_t)b * p.Nkv + hk) * p.Smax * 128) + c;
  constexpr int NU = 4; // keys per DPP row and trip (8 measured no better)
  // One trip = 64 keys per workgroup, 4 * NU per wave (NU per DPP row).  Split y takes trips y, y + splits, ...: the
  // splits differ by at most one trip whatever the length is, and the first trip's rows do not depend on the length
  // (a device scalar), so they are requested here, before anything else is read: the cache stream starts with the
  // launch.  Rows are clamped to the cache's last row; a trip past the end is read and never used (at most one per
  // workgroup).  Inside the loop the next trip is requested before this trip's arithmetic.
  i32x4 kw[NU], vw[NU], kn[NU], vn[NU];
  auto load_kv = [&](int base, i32x4 (&kd)[NU], i32x4 (&vd)[NU]) {
#pragma unroll
    for (int u = 0; u < NU; u++) {
      const int kk = min(base + u * 4 + g, p.Smax - 1);
      kd[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(kb + (int64_t)kk * 16));
      vd[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(vb + (int64_t)kk * 16));
    }
  };
  load_kv(blockIdx.y * 64 + wave * (4 * NU), kw, vw);
  const int len0 = *p.kv_len;
  const int L = max(0, min(len0 + p.kv_len_add, p.Smax));
  const int nk = (ROT && len0 >= 0 && len0 < p.Smax) ? len0 : -1; // cache position of the new token
  const int trips = (L + 63) >> 6;
  // the split whose trips contain the new token's position (wave-uniform)
  const bool has_new = ROT && nk >= 0 && nk < L && ((nk >> 6) % p.splits) == (int)blockIdx.y;

  float qf[8];
  i32x4 knew = {0, 0, 0, 0}, vnew = {0, 0, 0, 0};
  if (!ROT) {
    unpack8(reinterpret_cast<const uint4*>(p.q + (int64_t)bh * 128)[c], qf);
  } else {
    // chunk c holds first halves (c < 8) or second halves of the rotation pairs (h2, 64 + h2); partner chunk c ^ 8
    const bool first = c < 8;
    const int64_t pp = p.pos[p.B_pos == 1 ? 0 : b];
    const bool rot = p.emb != nullptr && pp >= 0 && pp < p.MP;
    float cs[8], sn[8];
#pragma unroll
    for (int e = 0; e < 8; e++)
      cs[e] = sn[e] = 0.f;
    if (rot) { // rows of 128 floats, 8 per chunk: 32-byte aligned
      const f32x4* cp = reinterpret_cast<const f32x4*>(p.emb + pp * 128 + (c & 7) * 8);
      const f32x4* sp = reinterpret_cast<const f32x4*>(p.emb + ((int64_t)p.MP + pp) * 128 + (c & 7) * 8);
      const f32x4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        cs[e] = c0[e];
        cs[4 + e] = c1[e];
        sn[e] = s0[e];
        sn[4 + e] = s1[e];
      }
    }
    auto rotate = [&](const uint16_t* row, float (&r)[8]) -> uint4 {
      const uint4 w = reinterpret_cast<const uint4*>(row)[c];
      if (!rot) {
        unpack8(w, r);
        return w;
      }
      const uint4 wo = reinterpret_cast<const uint4*>(row)[c ^ 8];
      float a[8], o[8];
      unpack8(w, a);
      unpack8(wo, o);
#pragma unroll
      for (int e = 0; e < 8; e++)
        r[e] = first ? a[e] * cs[e] - o[e] * sn[e] : a[e] * cs[e] + o[e] * sn[e];
      const uint4 out = pack8(r);
      unpack8(out, r); // the rotated row is a bf16 tensor
      return out;
    };
    rotate(p.q + (int64_t)bh * 128, qf);
    if (has_new) { // only the split that reads the new token's position needs its key and value
      float kr[8];
      const uint4 kw4 = rotate(p.k_new + ((int64_t)b * p.Nkv + hk) * 128, kr);
      knew = i32x4{(int)kw4.x, (int)kw4.y, (int)kw4.z, (int)kw4.w};
      vnew = *reinterpret_cast<const i32x4*>(p.v_new + ((int64_t)b * p.Nkv + hk) * 128 + c * 8);
      // one workgroup per KV head appends: the first query head of the group
      if (hq == hk * (p.Nq / p.Nkv) && tid < 16) {
        const int64_t o = (((int64_t)b * p.Nkv + hk) * p.Smax + nk) * 128 + c * 8;
        *reinterpret_cast<i32x4*>(const_cast<uint16_t*>(p.kc) + o) = knew;
        *reinterpret_cast<i32x4*>(const_cast<uint16_t*>(p.vc) + o) = vnew;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++)
    qf[e] *= p.scale;
  const uint16_t* mrow = p.mask ? p.mask + (int64_t)b * p.mask_ld : nullptr;

  float m = -3.0e38f, l = 0.f, acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++)
    acc[e] = 0.f;
  // the new token is not in the cache yet (or is being written by another workgroup right now): wherever its
  // position was read, the registers replace what the load returned
  auto patch_new = [&](int base, i32x4 (&kd)[NU], i32x4 (&vd)[NU]) {
    if (has_new) {
#pragma unroll
      for (int u = 0; u < NU; u++)
        if (base + u * 4 + g == nk) {
          kd[u] = knew;
          vd[u] = vnew;
        }
    }
  };
  patch_new(blockIdx.y * 64 + wave * (4 * NU), kw, vw);
  for (int t = blockIdx.y; t < trips; t += p.splits) {
    const int base = t * 64 + wave * (4 * NU);
    load_kv(base + p.splits * 64, kn, vn); // unconditional (rows are clamped): a branch here would drain the queue
    patch_new(base + p.splits * 64, kn, vn);
    int key[NU];
#pragma unroll
    for (int u = 0; u < NU; u++)
      key[u] = base + u * 4 + g;
    float sc[NU];
#pragma unroll
    for (int u = 0; u < NU; u++) {
      float kf[8];
      unpack8(as_uint4(kw[u]), kf);
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++)
        d = fmaf(qf[e], kf[e], d);
      d = row16_sum(d);
      if (mrow && key[u] < p.mask_ld && key[u] < L)
        d += bf16_bits_to_f32(mrow[key[u]]);
      sc[u] = key[u] < L ? d : -3.0e38f;
    }
    if (t * 64 + 64 > L) { // the last trip only (wave-uniform): rows past the end may hold anything, NaN included
#pragma unroll
      for (int u = 0; u < NU; u++)
        if (key[u] >= L)
          vw[u] = i32x4{0, 0, 0, 0};
    }
    float mn = m;
#pragma unroll
    for (int u = 0; u < NU; u++)
      mn = fmaxf(mn, sc[u]);
    const float alpha = __expf(m - mn);
    l *= alpha;
#pragma unroll
    for (int e = 0; e < 8; e++)
      acc[e] *= alpha;
#pragma unroll
    for (int u = 0; u < NU; u++) {
      const float pr = key[u] < L ? __expf(sc[u] - mn) : 0.f;
      l += pr;
      const float pb = round_bf16(pr);
      float vf[8];
      unpack8(as_uint4(vw[u]), vf);
#pragma unroll
      for (int e = 0; e < 8; e++)
        acc[e] = fmaf(pb, vf[e], acc[e]);
    }
    m = mn;
#pragma unroll
    for (int u = 0; u < NU; u++) {
      kw[u] = kn[u];
      vw[u] = vn[u];
    }
  }
  // merge the 16 (wave, row) states
  const int st = wave * 4 + g;
  if (c == 0) {
    sm[st] = m;
    sl[st] = l;
  }
#pragma unroll
  for (int e = 0; e < 8; e++)
    sacc[st][c * 8 + e] = acc[e];
  __syncthreads();
  float M = -3.0e38f, Ls = 0.f, o = 0.f;
  if (tid < 128) {
    M = sm[0];
#pragma unroll
    for (int i = 1; i < 16; i++)
      M = fmaxf(M, sm[i]);
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const float w = __expf(sm[i] - M);
      Ls = fmaf(w, sl[i], Ls);
      o = fmaf(w, sacc[i][tid], o);
    }
  }
  attn_finish(p, bh, tid, M, Ls, o);
}

// ---------------------------------------------------------------------------
// The same single-query attention for few trips per workgroup: at batch 1 the
// cache of one head is a few hundred KB, every workgroup makes one or two
// trips, and the vector arithmetic of the kernel above (bf16 unpacking, one
// multiply-add per element, a 16-lane reduction per 4 keys) costs more than
// the cache stream.  Here a lane owns an eighth (16 dims, chunks j*8 + q8) of
// FOUR keys per trip -- a wave instruction reads 8 whole rows, a wave covers
// 32 keys, the workgroup 128 -- and:
//   * q . k runs on v_dot2c_f32_bf16 (two bf16 products per instruction, no
//     unpacking), followed by an 8-lane reduction;
//   * the wave shares one running max (one exp per key and lane);
//   * p . v pairs the lane's keys: (v_a[e], v_b[e]) . (p_a, p_b), again on
//     the dot instruction, the pair assembled by one byte permute;
//   * the query is rotated once per workgroup (wave 0, one rotation pair per
//     lane) and handed to the lanes through LDS; the new key only in the
//     split that reads its position.
// The per-lane outputs (16 dims, partial over the lane's keys) are added up
// through LDS at the end.  The first trip's K and V rows (16 KB per wave) are
// requested before anything else; later trips request theirs when they start
// (the launch planner sends long loops to the kernel above).
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_mov<0xB1>(v));
  v = fmaxf(v, dpp_mov<0x4E>(v));
  v = fmaxf(v, dpp_mov<0x141>(v));
  v = fmaxf(v, dpp_mov<0x140>(v));
  const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

constexpr int ATTN_WIDE_KEYS = 128; // keys per workgroup and trip

template <bool ROT>
__global__ void __launch_bounds__(256, 4) // four workgroups per CU: at most 128 registers
attn_decode_wide_kernel(const AttnParams p) {
  __shared__ __align__(16) uint16_t q_s[128], k_s[128];
  __shared__ float sm[4], sl[4];
  __shared__ __align__(16) float sacc[4][8][132];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kq = lane >> 3, q8 = lane & 7;
  const int bh = blockIdx.x, b = bh / p.Nq, hq = bh - b * p.Nq;
  const int hk = hq / (p.Nq / p.Nkv);
  const int S = p.splits;
  const char* kb = reinterpret_cast<const char*>(p.kc + ((int64_t)b * p.Nkv + hk) * p.Smax * 128) + q8 * 16;
  const char* vb = reinterpret_cast<const char*>(p.vc + ((int64_t)b * p.Nkv + hk) * p.Smax * 128) + q8 * 16;
  // key set s of a trip: keys base + s*8 + kq; register [s][j] holds dims (j*8 + q8)*8 .. +7 as four bf16 pairs
  i32x4 kr[4][2], vr[4][2];
  auto load_rows = [&](const char* src, int base, i32x4 (&dst)[4][2]) {
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int key = min(base + s * 8 + kq, p.Smax - 1); // past the end: read, never used
#pragma unroll
      for (int j = 0; j < 2; j++)
        dst[s][j] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(src + (int64_t)key * 256 + j * 128));
    }
  };
  // A wave's loads return in the order of their issue.  Wave 0 prepares the query (and the new key): it asks for
  // those few values first, so that they do not queue behind its 16 KB of rows, and rotates them while the rows of
  // all four waves are on their way.  Lane i owns the rotation pair (i, 64 + i).
  i32x4 qp[2];
  float qx1 = 0.f, qx2 = 0.f, kx1 = 0.f, kx2 = 0.f, cs = 1.f, sn = 0.f;
  bool rot = false;
  if (!ROT) {
#pragma unroll
    for (int j = 0; j < 2; j++)
      qp[j] = reinterpret_cast<const i32x4*>(p.q + (int64_t)bh * 128)[j * 8 + q8];
  } else if (wave == 0) {
    const uint16_t* qrow = p.q + (int64_t)bh * 128;
    const uint16_t* krow = p.k_new + ((int64_t)b * p.Nkv + hk) * 128;
    qx1 = bf16_bits_to_f32(qrow[lane]);
    qx2 = bf16_bits_to_f32(qrow[64 + lane]);
    kx1 = bf16_bits_to_f32(krow[lane]);
    kx2 = bf16_bits_to_f32(krow[64 + lane]);
    const int64_t pp = p.pos[p.B_pos == 1 ? 0 : b];
    rot = p.emb != nullptr && pp >= 0 && pp < p.MP; // positions outside the table are left unrotated
    if (rot) {
      cs = p.emb[pp * 128 + lane];
      sn = p.emb[((int64_t)p.MP + pp) * 128 + lane];
    }
  }
  load_rows(kb, blockIdx.y * ATTN_WIDE_KEYS + wave * 32, kr);
  load_rows(vb, blockIdx.y * ATTN_WIDE_KEYS + wave * 32, vr);
  const int len0 = *p.kv_len;
  const int L = max(0, min(len0 + p.kv_len_add, p.Smax));
  const int nk = (ROT && len0 >= 0 && len0 < p.Smax) ? len0 : -1; // cache position of the new token
  const int trips = (L + ATTN_WIDE_KEYS - 1) / ATTN_WIDE_KEYS;
  // the split whose trips contain the new token's position (uniform over the workgroup)
  const bool has_new = ROT && nk >= 0 && nk < L && ((nk / ATTN_WIDE_KEYS) % S) == (int)blockIdx.y;

  if (ROT) {
    if (wave == 0) {
      q_s[lane] = (uint16_t)f32_to_bf16_bits(rot ? qx1 * cs - qx2 * sn : qx1);
      q_s[64 + lane] = (uint16_t)f32_to_bf16_bits(rot ? qx2 * cs + qx1 * sn : qx2);
      if (has_new) {
        k_s[lane] = (uint16_t)f32_to_bf16_bits(rot ? kx1 * cs - kx2 * sn : kx1);
        k_s[64 + lane] = (uint16_t)f32_to_bf16_bits(rot ? kx2 * cs + kx1 * sn : kx2);
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; j++)
      qp[j] = reinterpret_cast<const i32x4*>(q_s)[j * 8 + q8];
    // one workgroup per KV head appends: the first query head of the group, in the split that reads the position
    if (has_new && hq == hk * (p.Nq / p.Nkv) && tid < 16) {
      const int64_t o = (((int64_t)b * p.Nkv + hk) * p.Smax + nk) * 128 + tid * 8;
      *reinterpret_cast<i32x4*>(const_cast<uint16_t*>(p.kc) + o) = reinterpret_cast<const i32x4*>(k_s)[tid];
      *reinterpret_cast<i32x4*>(const_cast<uint16_t*>(p.vc) + o) =
          *reinterpret_cast<const i32x4*>(p.v_new + ((int64_t)b * p.Nkv + hk) * 128 + tid * 8);
    }
  }
  const uint16_t* mrow = p.mask ? p.mask + (int64_t)b * p.mask_ld : nullptr;

  float m = -3.0e38f, l = 0.f; // m is the same in every lane of the wave
  float acc[16];
#pragma unroll
  for (int e = 0; e < 16; e++)
    acc[e] = 0.f;
  for (int t = blockIdx.y; t < trips; t += S) {
    const int base = t * ATTN_WIDE_KEYS + wave * 32;
    if (t != (int)blockIdx.y) { // the workgroups of this kernel make few trips: no request queue across trips
      load_rows(kb, base, kr);
      load_rows(vb, base, vr);
    }
    if (has_new && nk >= base && nk < base + 32) {
      // the new token is not in the cache yet (or is being written right now): its lanes take the rotated key from
      // LDS and the value from the step's input
      const int s_new = (nk - base) >> 3;
      if (kq == ((nk - base) & 7)) {
#pragma unroll
        for (int s = 0; s < 4; s++)
          if (s == s_new) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
              kr[s][j] = reinterpret_cast<const i32x4*>(k_s)[j * 8 + q8];
              vr[s][j] = *reinterpret_cast<const i32x4*>(p.v_new + ((int64_t)b * p.Nkv + hk) * 128 + (j * 8 + q8) * 8);
            }
          }
      }
    }
    float sc[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int key = base + s * 8 + kq;
      float d = 0.f;
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          d = dot2_bf16((uint32_t)kr[s][j][r], (uint32_t)qp[j][r], d);
      d += dpp_mov<0xB1>(d);  // the eight parts of the key: quad_perm [1,0,3,2], [2,3,0,1], row_half_mirror
      d += dpp_mov<0x4E>(d);
      d += dpp_mov<0x141>(d);
      d *= p.scale;
      if (mrow && key < p.mask_ld && key < L)
        d += bf16_bits_to_f32(mrow[key]);
      sc[s] = key < L ? d : -3.0e38f;
    }
    const float mn = fmaxf(m, wave_max(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]))));
    if (mn > m) { // wave-uniform; rare once the first trips have passed
      const float alpha = __expf(m - mn);
      l *= alpha;
#pragma unroll
      for (int e = 0; e < 16; e++)
        acc[e] *= alpha;
      m = mn;
    }
    uint32_t pk[2] = {0, 0}; // probabilities of the key pairs (0, 1) and (2, 3) as packed bf16
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int key = base + s * 8 + kq;
      const float pr = key < L ? __expf(sc[s] - m) : 0.f;
      l += pr;
      pk[s >> 1] |= f32_to_bf16_bits(pr) << (16 * (s & 1));
      if (base + 32 > L && key >= L) { // rows past the end may hold anything, NaN included
#pragma unroll
        for (int j = 0; j < 2; j++)
          vr[s][j] = i32x4{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const uint32_t va = (uint32_t)vr[2 * h][j][r], vb2 = (uint32_t)vr[2 * h + 1][j][r];
          // v_perm_b32: selector bytes 0..3 pick from the second operand, 4..7 from the first
          const uint32_t lo = __builtin_amdgcn_perm(vb2, va, 0x05040100u); // (a.dim 2r, b.dim 2r)
          const uint32_t hi = __builtin_amdgcn_perm(vb2, va, 0x07060302u); // (a.dim 2r+1, b.dim 2r+1)
          acc[j * 8 + 2 * r] = dot2_bf16(lo, pk[h], acc[j * 8 + 2 * r]);
          acc[j * 8 + 2 * r + 1] = dot2_bf16(hi, pk[h], acc[j * 8 + 2 * r + 1]);
        }
  }
  // add up the lanes' partial outputs: [wave][kq][dim], rows padded against bank conflicts
#pragma unroll
  for (int j = 0; j < 2; j++) {
    float* dst = &sacc[wave][kq][(j * 8 + q8) * 8];
    *reinterpret_cast<f32x4*>(dst) = f32x4{acc[j * 8], acc[j * 8 + 1], acc[j * 8 + 2], acc[j * 8 + 3]};
    *reinterpret_cast<f32x4*>(dst + 4) = f32x4{acc[j * 8 + 4], acc[j * 8 + 5], acc[j * 8 + 6], acc[j * 8 + 7]};
  }
  // every key's l sits in the eight lanes of the key: the wave sum counts it eight times (exactly, a power of two)
  const float lw = wave_sum(l) * 0.125f;
  if (lane == 0) {
    sm[wave] = m;
    sl[wave] = lw;
  }
  __syncthreads();
  float M = -3.0e38f, Ls = 0.f, o = 0.f;
  if (tid < 128) {
    M = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
#pragma unroll
    for (int w = 0; w < 4; w++) {
      float so = 0.f;
#pragma unroll
      for (int i = 0; i < 8; i++)
        so += sacc[w][i][tid];
      const float wt = __expf(sm[w] - M);
      Ls = fmaf(wt, sl[w], Ls);
      o = fmaf(wt, so, o);
    }
  }
  attn_finish(p, bh, tid, M, Ls, o);
}

__global__ void __launch_bounds__(128)
attn_combine_kernel(const AttnParams p) {
  const int bh = blockIdx.x, tid = threadIdx.x;
  const float* src = p.part + (int64_t)bh * p.splits * 130;
  float M = -3.0e38f;
  for (int i = 0; i < p.splits; i++)
    M = fmaxf(M, src[i * 130]);
  float Ls = 0.f, o = 0.f;
  for (int i = 0; i < p.splits; i++) {
    const float w = __expf(src[i * 130] - M);
    Ls = fmaf(w, src[i * 130 + 1], Ls);
    o = fmaf(w, src[i * 130 + 2 + tid], o);
  }
  p.out[(int64_t)bh * 128 + tid] = (uint16_t)f32_to_bf16_bits(Ls > 0.f ? o / Ls : 0.f);
}

// ---------------------------------------------------------------------------
// Prompt attention: S query tokens per sequence at positions past .. past+S-1
// over the cache [B][Nkv][Smax][128], causal (query i sees keys 0 .. past+i).
// Grid (ceil(S/64), B*Nq); 4 waves of 16 queries each share the K and V tiles
// of 64 keys through LDS.  Both products run on the 16x16x32 bf16 MFMA in
// transposed form, so that no probability ever changes lanes:
//   scores^T[key][query] = K tile (rows = keys) x Q^T      (4 MFMAs per 16 keys)
//   out^T[dim][query]   += V^T tile (rows = dims) x P^T    (2 MFMAs per 16 dims)
// The score tile's result layout -- lane (g, c) holds keys g*4+r of query c --
// is, after rounding to bf16, already the second operand of the V product
// (its 32 K slots filled with the lane's keys of two score tiles; the V^T
// operand picks the same keys).  V is transposed on its way into LDS.
// Online softmax per query: fp32 scores * 1/sqrt(H) + mask, running max and
// sum, probabilities rounded to bf16 before they multiply V, sum and output
// in fp32 (the same arithmetic as the single-query kernel above).
// ---------------------------------------------------------------------------
struct AttnPrefillParams {
  const uint16_t* q;    // [B][S][Nq][128]
  const uint16_t* kc;   // [B][Nkv][Smax][128]
  const uint16_t* vc;
  const uint16_t* mask; // bf16 [B][mask_ld] additive, or null
  uint16_t* out;        // [B][S][Nq][128]
  int B, S, Nq, Nkv, Smax, mask_ld, past;
  float scale;
  int H;                // head size (attn_prefill_hd_kernel; the kernel for 128 does not read it)
};

constexpr int AP_KP = 136; // LDS row pitch of the K tile, bf16 elements (128 + 8: rows 16-byte aligned, banks spread)
constexpr int AP_VP = 68;  // LDS row pitch of the V^T tile (64 keys + 4: rows 8-byte aligned)

// QG = query groups of 16 per wave: every K / V^T operand read from LDS feeds QG MFMAs (with one group the LDS
// reads, 32 KB per wave and key tile, take twice the cycles of the 32 MFMAs they feed).
template <int QG>
__global__ void __launch_bounds__(256)
attn_prefill_kernel(const AttnPrefillParams p) {
  __shared__ __align__(16) uint16_t ks[64 * AP_KP];
  __shared__ __align__(16) uint16_t vt[128 * AP_VP];
  constexpr int QB = 64 * QG; // queries per workgroup
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, c = lane & 15;
  const int bh = blockIdx.y, b = bh / p.Nq, hq = bh - b * p.Nq;
  const int hk = hq / (p.Nq / p.Nkv);
  // The last query blocks see the most keys: start them first.  Two workgroups share a CU, and the dispatcher puts
  // workgroup i + 256 beside workgroup i: the heads of every other run of 256 workgroups walk their query blocks
  // the other way round, so that a long block meets a short one instead of its twin of another head.  (One order
  // per head -- taken from the head's first workgroup -- or a run boundary inside a head would visit some blocks
  // twice and others never.)
  const int wg0 = (int)(blockIdx.y * gridDim.x);
  const int qblk = ((wg0 >> 8) & 1) ? (int)blockIdx.x : (int)gridDim.x - 1 - (int)blockIdx.x;
  const int q0 = qblk * QB + wave * (16 * QG);
  const int last_key = p.past + p.S - 1;

  int qpos[QG]; // last key this lane's query of group qg sees (rows past the end repeat the last query, never stored)
  bf16x8 qreg[QG][4];
#pragma unroll
  for (int qg = 0; qg < QG; qg++) {
    const int qi = min(q0 + qg * 16 + c, p.S - 1);
    qpos[qg] = p.past + qi;
    const uint16_t* qrow = p.q + (((int64_t)b * p.S + qi) * p.Nq + hq) * 128;
#pragma unroll
    for (int j = 0; j < 4; j++)
      qreg[qg][j] = *reinterpret_cast<const bf16x8*>(qrow + j * 32 + g * 8);
  }
  const uint16_t* kbase = p.kc + ((int64_t)b * p.Nkv + hk) * p.Smax * 128;
  const uint16_t* vbase = p.vc + ((int64_t)b * p.Nkv + hk) * p.Smax * 128;
  const uint16_t* mrow = p.mask ? p.mask + (int64_t)b * p.mask_ld : nullptr;

  // staging registers: K rows chunk-fastest (coalesced); V: a thread takes one 16-byte chunk (8 dims) of FOUR
  // consecutive keys, so that the transposed image is written as 8 x 8 bytes (4 keys of one dim, packed with two
  // byte permutes) instead of 32 two-byte writes
  i32x4 kst[4], vst[4];
  const int vq = tid & 15, vch = tid >> 4; // key quad, chunk
  auto load_tile = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int idx = tid + i * 256;
      const int kk = min(kb * 64 + (idx >> 4), last_key);
      kst[i] = *reinterpret_cast<const i32x4*>(kbase + (int64_t)kk * 128 + (idx & 15) * 8);
      const int kv = min(kb * 64 + vq * 4 + i, last_key);
      vst[i] = *reinterpret_cast<const i32x4*>(vbase + (int64_t)kv * 128 + vch * 8);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int idx = tid + i * 256;
      *reinterpret_cast<i32x4*>(ks + (idx >> 4) * AP_KP + (idx & 15) * 8) = kst[i];
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
      // dim vch*8 + e of keys 4*vq .. 4*vq+3: the low (e even) or high (e odd) halves of dword e/2 of the four rows
      const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
      const uint32_t lo = __builtin_amdgcn_perm((uint32_t)vst[1][e >> 1], (uint32_t)vst[0][e >> 1], sel);
      const uint32_t hi = __builtin_amdgcn_perm((uint32_t)vst[3][e >> 1], (uint32_t)vst[2][e >> 1], sel);
      *reinterpret_cast<uint2*>(vt + (vch * 8 + e) * AP_VP + vq * 4) = make_uint2(lo, hi);
    }
  };

  const float scale2 = p.scale * 1.44269504f;
  float m[QG], l[QG];
  f32x4 acc[QG][8];
#pragma unroll
  for (int qg = 0; qg < QG; qg++) {
    m[qg] = -3.0e38f;
    l[qg] = 0.f;
#pragma unroll
    for (int dt = 0; dt < 8; dt++)
      acc[qg][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // key tiles up to the one holding the last key of the workgroup's last query (the same for all four waves)
  const int nkb = (p.past + min(qblk * QB + QB - 1, p.S - 1)) / 64 + 1;
  load_tile(0);
  for (int kb = 0; kb < nkb; kb++) {
    __syncthreads(); // the previous tile has been read by every wave
    store_tile();
    __syncthreads();
    if (kb + 1 < nkb)
      load_tile(kb + 1); // in flight during the arithmetic below

    f32x4 sc[QG][4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
#pragma unroll
      for (int qg = 0; qg < QG; qg++)
        sc[qg][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(ks + (t * 16 + c) * AP_KP + j * 32 + g * 8);
#pragma unroll
        for (int qg = 0; qg < QG; qg++)
          sc[qg][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qreg[qg][j], sc[qg][t], 0, 0, 0);
      }
    }
    // Scores in the base-2 domain (scale * log2 e folded into one multiplier): a probability is one exp2.  The
    // additive mask is read only when there is one (wave-uniform branch: no addresses, no predicated loads).
#pragma unroll
    for (int qg = 0; qg < QG; qg++)
#pragma unroll
      for (int t = 0; t < 4; t++)
        sc[qg][t] *= scale2;
    if (mrow) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int key = kb * 64 + (i >> 2) * 16 + g * 4 + (i & 3);
        const float mk = key < p.mask_ld ? bf16_bits_to_f32(mrow[key]) * 1.44269504f : 0.f;
#pragma unroll
        for (int qg = 0; qg < QG; qg++)
          sc[qg][i >> 2][i & 3] += mk;
      }
    }
    bf16x8 pb[QG][2];
    // only the tiles that reach past the position of this wave's first query hide anything (wave-uniform)
    const bool edge = kb * 64 + 63 > p.past + q0;
#pragma unroll
    for (int qg = 0; qg < QG; qg++) {
      if (edge) {
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int key = kb * 64 + t * 16 + g * 4 + r;
            // keys past the causal edge get -inf, whose exp2 is exactly 0 against the finite running maximum
            sc[qg][t][r] = key <= qpos[qg] ? sc[qg][t][r] : -INFINITY;
          }
      }
      float mx = -3.0e38f;
#pragma unroll
      for (int t = 0; t < 4; t++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          mx = fmaxf(mx, sc[qg][t][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float mn = fmaxf(m[qg], mx); // finite from the first tile on: key 0 is visible to every query
      const float alpha = __builtin_amdgcn_exp2f(m[qg] - mn);
      l[qg] *= alpha;
#pragma unroll
      for (int dt = 0; dt < 8; dt++)
        acc[qg][dt] *= alpha;
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const float pr = __builtin_amdgcn_exp2f(sc[qg][2 * u + (j >> 2)][j & 3] - mn);
          l[qg] += pr;
          pb[qg][u][j] = (__bf16)pr;
        }
      m[qg] = mn;
    }
#pragma unroll
    for (int dt = 0; dt < 8; dt++)
#pragma unroll
      for (int u = 0; u < 2; u++) {
        // K slots g*8 .. g*8+7 of the operand = keys u*32 + g*4 .. +3 and u*32 + 16 + g*4 .. +3 of the tile,
        // the keys pb[.][u] holds in the same slots
        const uint16_t* vrow = vt + (dt * 16 + c) * AP_VP + u * 32 + g * 4;
        const uint2 lo = *reinterpret_cast<const uint2*>(vrow), hi = *reinterpret_cast<const uint2*>(vrow + 16);
        const i32x4 av = {(int)lo.x, (int)lo.y, (int)hi.x, (int)hi.y};
#pragma unroll
        for (int qg = 0; qg < QG; qg++)
          acc[qg][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), pb[qg][u], acc[qg][dt], 0, 0, 0);
      }
  }
#pragma unroll
  for (int qg = 0; qg < QG; qg++) {
    float ls = l[qg];
    ls += __shfl_xor(ls, 16);
    ls += __shfl_xor(ls, 32);
    const int qi = q0 + qg * 16 + c;
    if (qi < p.S) {
      uint16_t* orow = p.out + (((int64_t)b * p.S + qi) * p.Nq + hq) * 128;
#pragma unroll
      for (int dt = 0; dt < 8; dt++) {
        uint32_t w[2];
#pragma unroll
        for (int h = 0; h < 2; h++)
          w[h] = f32_to_bf16_bits(ls > 0.f ? acc[qg][dt][2 * h] / ls : 0.f) |
                 (f32_to_bf16_bits(ls > 0.f ? acc[qg][dt][2 * h + 1] / ls : 0.f) << 16);
        *reinterpret_cast<uint2*>(orow + dt * 16 + g * 4) = make_uint2(w[0], w[1]);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Prompt attention at head sizes other than 128: attn_prefill_kernel with the head size padded to HD = 64, 128 or
// 256 (H a multiple of 8, H <= HD; dims past H are staged as zeros and not stored), the K tile 64 x (HD + 8) and the
// V^T tile HD x 68 in dynamic LDS, HD / 32 MFMAs per 16 keys for the scores and HD / 16 output tiles per query group.
// Same arithmetic and rounding points as the kernel for 128.
// ---------------------------------------------------------------------------
template <int QG, int HD>
__global__ void __launch_bounds__(256)
attn_prefill_hd_kernel(const AttnPrefillParams p) {
  extern __shared__ __align__(16) uint16_t ap_lds[];
  constexpr int KP = HD + 8, VP = AP_VP, NJ = HD / 32, NDT = HD / 16, CH = HD / 8;
  constexpr int VI = (CH + 15) / 16; // value chunks per thread: 16 threads (key quads) x 16 chunks per pass
  uint16_t* ks = ap_lds;           // [64 keys][KP]
  uint16_t* vt = ap_lds + 64 * KP; // [HD dims][VP]
  constexpr int QB = 64 * QG;
  const int H = p.H, HC = H >> 3;  // real 8-dim chunks per row
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, c = lane & 15;
  const int bh = blockIdx.y, b = bh / p.Nq, hq = bh - b * p.Nq;
  const int hk = hq / (p.Nq / p.Nkv);
  // the last query blocks see the most keys: start them first; the heads of every other run of 256 workgroups the
  // other way round, so that the workgroups that share a CU (i, i + 256, ...) are a long one and a short one (one
  // order per head, taken from the head's first workgroup)
  const int wg0 = (int)(blockIdx.y * gridDim.x);
  const int qblk = ((wg0 >> 8) & 1) ? (int)blockIdx.x : (int)gridDim.x - 1 - (int)blockIdx.x;
  const int q0 = qblk * QB + wave * (16 * QG);
  const int last_key = p.past + p.S - 1;
  const i32x4 zero4 = {0, 0, 0, 0};

  int qpos[QG];
  bf16x8 qreg[QG][NJ];
#pragma unroll
  for (int qg = 0; qg < QG; qg++) {
    const int qi = min(q0 + qg * 16 + c, p.S - 1);
    qpos[qg] = p.past + qi;
    const uint16_t* qrow = p.q + (((int64_t)b * p.S + qi) * p.Nq + hq) * H;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
      const int ch = j * 4 + g;
      qreg[qg][j] = __builtin_bit_cast(bf16x8, ch < HC ? *reinterpret_cast<const i32x4*>(qrow + ch * 8) : zero4);
    }
  }
  const uint16_t* kbase = p.kc + ((int64_t)b * p.Nkv + hk) * (int64_t)p.Smax * H;
  const uint16_t* vbase = p.vc + ((int64_t)b * p.Nkv + hk) * (int64_t)p.Smax * H;
  const uint16_t* mrow = p.mask ? p.mask + (int64_t)b * p.mask_ld : nullptr;

  // staging registers: K rows chunk-fastest; V: a thread takes one chunk of FOUR consecutive keys per pass
  i32x4 kst[NJ], vst[VI][4];
  const int vq = tid & 15;
  auto load_tile = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NJ; i++) {
      const int idx = tid + i * 256;
      const int key = idx / CH, ch = idx % CH;
      const int kk = min(kb * 64 + key, last_key);
      kst[i] = ch < HC ? *reinterpret_cast<const i32x4*>(kbase + (int64_t)kk * H + ch * 8) : zero4;
    }
#pragma unroll
    for (int it = 0; it < VI; it++) {
      const int vch = (tid >> 4) + it * 16;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int kv = min(kb * 64 + vq * 4 + i, last_key);
        vst[it][i] = vch < HC ? *reinterpret_cast<const i32x4*>(vbase + (int64_t)kv * H + vch * 8) : zero4;
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < NJ; i++) {
      const int idx = tid + i * 256;
      *reinterpret_cast<i32x4*>(ks + (idx / CH) * KP + (idx % CH) * 8) = kst[i];
    }
#pragma unroll
    for (int it = 0; it < VI; it++) {
      const int vch = (tid >> 4) + it * 16;
      if (vch < CH) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
          const uint32_t lo = __builtin_amdgcn_perm((uint32_t)vst[it][1][e >> 1], (uint32_t)vst[it][0][e >> 1], sel);
          const uint32_t hi = __builtin_amdgcn_perm((uint32_t)vst[it][3][e >> 1], (uint32_t)vst[it][2][e >> 1], sel);
          *reinterpret_cast<uint2*>(vt + (vch * 8 + e) * VP + vq * 4) = make_uint2(lo, hi);
        }
      }
    }
  };

  const float scale2 = p.scale * 1.44269504f;
  float m[QG], l[QG];
  f32x4 acc[QG][NDT];
#pragma unroll
  for (int qg = 0; qg < QG; qg++) {
    m[qg] = -3.0e38f;
    l[qg] = 0.f;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
      acc[qg][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int nkb = (p.past + min(qblk * QB + QB - 1, p.S - 1)) / 64 + 1;
  load_tile(0);
  for (int kb = 0; kb < nkb; kb++) {
    __syncthreads(); // the previous tile has been read by every wave
    store_tile();
    __syncthreads();
    if (kb + 1 < nkb)
      load_tile(kb + 1); // in flight during the arithmetic below

    f32x4 sc[QG][4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
#pragma unroll
      for (int qg = 0; qg < QG; qg++)
        sc[qg][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(ks + (t * 16 + c) * KP + j * 32 + g * 8);
#pragma unroll
        for (int qg = 0; qg < QG; qg++)
          sc[qg][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qreg[qg][j], sc[qg][t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int qg = 0; qg < QG; qg++)
#pragma unroll
      for (int t = 0; t < 4; t++)
        sc[qg][t] *= scale2;
    if (mrow) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int key = kb * 64 + (i >> 2) * 16 + g * 4 + (i & 3);
        const float mk = key < p.mask_ld ? bf16_bits_to_f32(mrow[key]) * 1.44269504f : 0.f;
#pragma unroll
        for (int qg = 0; qg < QG; qg++)
          sc[qg][i >> 2][i & 3] += mk;
      }
    }
    bf16x8 pb[QG][2];
    const bool edge = kb * 64 + 63 > p.past + q0;
#pragma unroll
    for (int qg = 0; qg < QG; qg++) {
      if (edge) {
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int key = kb * 64 + t * 16 + g * 4 + r;
            sc[qg][t][r] = key <= qpos[qg] ? sc[qg][t][r] : -INFINITY;
          }
      }
      float mx = -3.0e38f;
#pragma unroll
      for (int t = 0; t < 4; t++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          mx = fmaxf(mx, sc[qg][t][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float mn = fmaxf(m[qg], mx);
      const float alpha = __builtin_amdgcn_exp2f(m[qg] - mn);
      l[qg] *= alpha;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++)
        acc[qg][dt] *= alpha;
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const float pr = __builtin_amdgcn_exp2f(sc[qg][2 * u + (j >> 2)][j & 3] - mn);
          l[qg] += pr;
          pb[qg][u][j] = (__bf16)pr;
        }
      m[qg] = mn;
    }
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const uint16_t* vrow = vt + (dt * 16 + c) * VP + u * 32 + g * 4;
        const uint2 lo = *reinterpret_cast<const uint2*>(vrow), hi = *reinterpret_cast<const uint2*>(vrow + 16);
        const i32x4 av = {(int)lo.x, (int)lo.y, (int)hi.x, (int)hi.y};
#pragma unroll
        for (int qg = 0; qg < QG; qg++)
          acc[qg][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), pb[qg][u], acc[qg][dt], 0, 0, 0);
      }
  }
#pragma unroll
  for (int qg = 0; qg < QG; qg++) {
    float ls = l[qg];
    ls += __shfl_xor(ls, 16);
    ls += __shfl_xor(ls, 32);
    const int qi = q0 + qg * 16 + c;
    if (qi < p.S) {
      uint16_t* orow = p.out + (((int64_t)b * p.S + qi) * p.Nq + hq) * H;
#pragma unroll
      for (int dt = 0; dt < NDT; dt++) {
        if (dt * 16 + g * 4 < H) { // H is a multiple of 8: the four dims of this lane exist together
          uint32_t w[2];
#pragma unroll
          for (int h = 0; h < 2; h++)
            w[h] = f32_to_bf16_bits(ls > 0.f ? acc[qg][dt][2 * h] / ls : 0.f) |
                   (f32_to_bf16_bits(ls > 0.f ? acc[qg][dt][2 * h + 1] / ls : 0.f) << 16);
          *reinterpret_cast<uint2*>(orow + dt * 16 + g * 4) = make_uint2(w[0], w[1]);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Greedy step of a generation loop: next token = argmax of the row's logits (the first maximal index; a NaN counts
// as maximal, as torch.argmax has it), stored as int64; the position of the row moves on by one; the token's
// embedding row becomes the row of the next step's hidden states; workgroup 0 moves the cache length on by one.
// One workgroup of 1024 threads per row: 16-byte loads, (value, index) maxima through DPP-free LDS steps.
// ---------------------------------------------------------------------------
struct GreedyKey {
  float v;
  int i;
};
__device__ __forceinline__ bool greedy_before(float v, int i, float bv, int bi) {
  // total order: NaN above everything, then larger value, then smaller index
  const bool vn = v != v, bn = bv != bv;
  if (vn != bn)
    return vn;
  if (!vn && v != bv)
    return v > bv;
  return i < bi;
}

__global__ void __launch_bounds__(1024)
greedy_next_kernel(const uint16_t* __restrict__ logits, int V, const uint16_t* __restrict__ embed, int hidden,
                   int64_t* __restrict__ tokens, int64_t* __restrict__ pos, int32_t* __restrict__ seq_len,
                   uint16_t* __restrict__ h_next) {
  __shared__ float sv[1024];
  __shared__ int si[1024];
  const int b = blockIdx.x, tid = threadIdx.x;
  const uint16_t* row = logits + (size_t)b * V;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = tid * 8; c < V; c += 1024 * 8) { // V % 8 == 0
    const uint4 raw = *reinterpret_cast<const uint4*>(row + c);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float v = bf16_bits_to_f32((w[e >> 1] >> ((e & 1) * 16)) & 0xffffu);
      if (greedy_before(v, c + e, bv, bi)) {
        bv = v;
        bi = c + e;
      }
    }
  }
  sv[tid] = bv;
  si[tid] = bi;
  __syncthreads();
  for (int step = 512; step > 0; step >>= 1) {
    if (tid < step && greedy_before(sv[tid + step], si[tid + step], sv[tid], si[tid])) {
      sv[tid] = sv[tid + step];
      si[tid] = si[tid + step];
    }
    __syncthreads();
  }
  const int tok = si[0];
  if (tid == 0) {
    tokens[b] = tok;
    if (pos)
      pos[b] += 1;
    if (seq_len && b == 0)
      seq_len[0] += 1;
  }
  if (h_next)
    for (int c = tid * 8; c < hidden; c += 1024 * 8) // hidden % 8 == 0
      *reinterpret_cast<uint4*>(h_next + (size_t)b * hidden + c) = *reinterpret_cast<const uint4*>(embed + (size_t)tok * hidden + c);
}

} // namespace tppx

using namespace tppx;

extern "C" int tppx_greedy_next(const void* logits, int64_t B, int64_t V, const void* embed, int64_t hidden, void* tokens,
                                void* pos, void* seq_len, void* h_next, tppx_stream_t stream) {
  const char* who = "tppx_greedy_next";
  TPPX_REQUIRE(logits && tokens, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(logits), TPPX_EINVAL, "%s: logits not 16-byte aligned", who);
  TPPX_REQUIRE(B > 0 && B < (1 << 16) && V > 0 && V % 8 == 0 && V < ((int64_t)1 << 31), TPPX_ESHAPE,
               "%s: bad shape B=%ld V=%ld (V must be a multiple of 8)", who, (long)B, (long)V);
  TPPX_REQUIRE(!h_next || (embed && aligned16(embed) && aligned16(h_next) && hidden > 0 && hidden % 8 == 0), TPPX_EINVAL,
               "%s: the next hidden states need a 16-byte aligned embedding table and output with hidden %% 8 == 0", who);
  greedy_next_kernel<<<dim3((unsigned)B), dim3(1024), 0, (hipStream_t)stream>>>(
      (const uint16_t*)logits, (int)V, (const uint16_t*)embed, (int)hidden, (int64_t*)tokens, (int64_t*)pos, (int32_t*)seq_len,
      (uint16_t*)h_next);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_rms_norm(const void* x, const void* gamma, int gamma_dtype, void* y, int64_t rows, int64_t K,
                             float eps, tppx_stream_t stream) {
  TPPX_REQUIRE(x && gamma && y, TPPX_EINVAL, "tppx_rms_norm: null pointer");
  TPPX_REQUIRE(aligned16(x) && aligned16(gamma) && aligned16(y), TPPX_EINVAL, "tppx_rms_norm: pointer not 16-byte aligned");
  TPPX_REQUIRE(gamma_dtype == TPPX_DT_F32 || gamma_dtype == TPPX_DT_BF16, TPPX_EINVAL, "tppx_rms_norm: unknown gamma dtype %d", gamma_dtype);
  TPPX_REQUIRE(rows > 0 && rows < ((int64_t)1 << 31) && K > 0 && K % 8 == 0 && K < (1 << 24), TPPX_ESHAPE,
               "tppx_rms_norm: bad shape rows=%ld K=%ld (K must be a multiple of 8)", (long)rows, (long)K);
  if (gamma_dtype == TPPX_DT_F32)
    rms_norm_kernel<true><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
        (const uint16_t*)x, gamma, (uint16_t*)y, (int)K, eps);
  else
    rms_norm_kernel<false><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
        (const uint16_t*)x, gamma, (uint16_t*)y, (int)K, eps);
  return check_hip(hipGetLastError(), "tppx_rms_norm");
}

extern "C" int tppx_layer_norm(const void* x, const void* gamma, const void* beta, int param_dtype, void* y,
                               int64_t rows, int64_t K, float eps, tppx_stream_t stream) {
  TPPX_REQUIRE(x && gamma && beta && y, TPPX_EINVAL, "tppx_layer_norm: null pointer");
  TPPX_REQUIRE(aligned16(x) && aligned16(gamma) && aligned16(beta) && aligned16(y), TPPX_EINVAL,
               "tppx_layer_norm: pointer not 16-byte aligned");
  TPPX_REQUIRE(param_dtype == TPPX_DT_F32 || param_dtype == TPPX_DT_BF16, TPPX_EINVAL,
               "tppx_layer_norm: unknown gamma / beta dtype %d", param_dtype);
  TPPX_REQUIRE(rows > 0 && rows < ((int64_t)1 << 31) && K > 0 && K % 8 == 0 && K < (1 << 24), TPPX_ESHAPE,
               "tppx_layer_norm: bad shape rows=%ld K=%ld (K must be a multiple of 8)", (long)rows, (long)K);
  if (param_dtype == TPPX_DT_F32)
    layer_norm_kernel<true><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
        (const uint16_t*)x, gamma, beta, (uint16_t*)y, (int)K, eps);
  else
    layer_norm_kernel<false><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(
        (const uint16_t*)x, gamma, beta, (uint16_t*)y, (int)K, eps);
  return check_hip(hipGetLastError(), "tppx_layer_norm");
}

static int rotary_common(const char* who, RotaryParams& p, hipStream_t stream) {
  TPPX_REQUIRE(p.B > 0 && p.S > 0 && p.H >= 8 && p.H <= 512 && p.H % 8 == 0, TPPX_ESHAPE,
               "%s: bad shape B=%d S=%d H=%d (head size must be a multiple of 8 up to 512)", who, p.B, p.S, p.H);
  if (p.emb)
    TPPX_REQUIRE(p.HR > 0 && p.HR <= p.H && p.HR % 16 == 0 && p.MP > 0, TPPX_ESHAPE,
                 "%s: rotary_dim=%d must be a multiple of 16 and <= H=%d", who, p.HR, p.H);
  TPPX_REQUIRE(p.B_pos == 1 || p.B_pos == p.B, TPPX_ESHAPE, "%s: position_ids shape not compatible", who);
  const int heads = (p.q ? p.Nq : 0) + (p.k ? p.Nkv : 0) + ((p.v && p.vc) ? p.Nkv : 0);
  const int64_t total = (int64_t)p.B * p.S * heads * (p.H / 8);
  TPPX_REQUIRE(total > 0 && total < ((int64_t)1 << 40), TPPX_ESHAPE, "%s: nothing to do", who);
  rotary_append_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream>>>(p);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_rotary_llama(void* t, const void* emb_pos, const void* pos, int64_t B, int64_t S, int64_t N,
                                 int64_t H, int64_t MP, int64_t HR, int64_t B_pos, tppx_stream_t stream) {
  TPPX_REQUIRE(t && emb_pos && pos, TPPX_EINVAL, "tppx_rotary_llama: null pointer");
  TPPX_REQUIRE(aligned16(t), TPPX_EINVAL, "tppx_rotary_llama: pointer not 16-byte aligned");
  TPPX_REQUIRE(N > 0, TPPX_ESHAPE, "tppx_rotary_llama: N=%ld", (long)N);
  RotaryParams p;
  memset(&p, 0, sizeof(p));
  p.q = (uint16_t*)t;
  p.emb = (const float*)emb_pos;
  p.pos = (const int64_t*)pos;
  p.B = (int)B; p.S = (int)S; p.Nq = (int)N; p.H = (int)H; p.MP = (int)MP; p.HR = (int)HR; p.B_pos = (int)B_pos;
  return rotary_common("tppx_rotary_llama", p, (hipStream_t)stream);
}

extern "C" int tppx_rotary_kv_append_llama(void* q, void* k, const void* v, const void* emb_pos, const void* pos,
                                           void* kcache, void* vcache, const void* offset_dev, int64_t B,
                                           int64_t S, int64_t Nq, int64_t Nkv, int64_t H, int64_t MP, int64_t HR,
                                           int64_t B_pos, int64_t Smax, tppx_stream_t stream) {
  const char* who = "tppx_rotary_kv_append_llama";
  TPPX_REQUIRE(k && v && kcache && vcache && offset_dev && pos, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(k) && aligned16(v) && aligned16(kcache) && aligned16(vcache) && (!q || aligned16(q)),
               TPPX_EINVAL, "%s: pointer not 16-byte aligned", who);
  TPPX_REQUIRE(Nkv > 0 && Smax > 0 && (!q || Nq > 0), TPPX_ESHAPE, "%s: bad head counts / capacity", who);
  RotaryParams p;
  memset(&p, 0, sizeof(p));
  p.q = (uint16_t*)q; p.k = (uint16_t*)k; p.v = (const uint16_t*)v;
  p.kc = (uint16_t*)kcache; p.vc = (uint16_t*)vcache;
  p.emb = (const float*)emb_pos; p.pos = (const int64_t*)pos; p.offset = (const int32_t*)offset_dev;
  p.B = (int)B; p.S = (int)S; p.Nq = (int)Nq; p.Nkv = (int)Nkv; p.H = (int)H; p.MP = (int)MP; p.HR = (int)HR;
  p.B_pos = (int)B_pos; p.Smax = (int)Smax;
  return rotary_common(who, p, (hipStream_t)stream);
}

extern "C" int tppx_rotary_gptj(void* t, const void* emb_pos, const void* pos, int64_t B, int64_t S, int64_t N,
                                int64_t H, int64_t MP, int64_t HR, int64_t B_pos, tppx_stream_t stream) {
  TPPX_REQUIRE(t && emb_pos && pos, TPPX_EINVAL, "tppx_rotary_gptj: null pointer");
  TPPX_REQUIRE(aligned16(t), TPPX_EINVAL, "tppx_rotary_gptj: pointer not 16-byte aligned");
  TPPX_REQUIRE(N > 0, TPPX_ESHAPE, "tppx_rotary_gptj: N=%ld", (long)N);
  RotaryParams p;
  memset(&p, 0, sizeof(p));
  p.q = (uint16_t*)t;
  p.emb = (const float*)emb_pos;
  p.pos = (const int64_t*)pos;
  p.B = (int)B; p.S = (int)S; p.Nq = (int)N; p.H = (int)H; p.MP = (int)MP; p.HR = (int)HR; p.B_pos = (int)B_pos;
  p.gptj = 1;
  return rotary_common("tppx_rotary_gptj", p, (hipStream_t)stream);
}

extern "C" int tppx_rotary_kv_append_gptj(void* q, void* k, const void* v, const void* emb_pos, const void* pos,
                                          void* kcache, void* vcache, const void* offset_dev, int64_t B, int64_t S,
                                          int64_t Nq, int64_t Nkv, int64_t H, int64_t MP, int64_t HR, int64_t B_pos,
                                          int64_t Smax, tppx_stream_t stream) {
  const char* who = "tppx_rotary_kv_append_gptj";
  TPPX_REQUIRE(k && v && kcache && vcache && offset_dev && pos && emb_pos, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(k) && aligned16(v) && aligned16(kcache) && aligned16(vcache) && (!q || aligned16(q)),
               TPPX_EINVAL, "%s: pointer not 16-byte aligned", who);
  TPPX_REQUIRE(Nkv > 0 && Smax > 0 && (!q || Nq > 0), TPPX_ESHAPE, "%s: bad head counts / capacity", who);
  RotaryParams p;
  memset(&p, 0, sizeof(p));
  p.q = (uint16_t*)q; p.k = (uint16_t*)k; p.v = (const uint16_t*)v;
  p.kc = (uint16_t*)kcache; p.vc = (uint16_t*)vcache;
  p.emb = (const float*)emb_pos; p.pos = (const int64_t*)pos; p.offset = (const int32_t*)offset_dev;
  p.B = (int)B; p.S = (int)S; p.Nq = (int)Nq; p.Nkv = (int)Nkv; p.H = (int)H; p.MP = (int)MP; p.HR = (int)HR;
  p.B_pos = (int)B_pos; p.Smax = (int)Smax;
  p.gptj = 1;
  return rotary_common(who, p, (hipStream_t)stream);
}

// shared tail of the two single-query entry points: split planning, counters, launch
static int attn_decode_launch(const char* who, AttnParams& p, bool rot, int64_t B, int64_t Nq, int64_t Smax, void* ws,
                              int64_t ws_bytes, hipStream_t stream) {
  // The wide kernel (128 keys per workgroup and trip) is the default: measured against the row kernel (64 keys per
  // trip) over 32 heads, it is faster at every batch size from 1 to 64 and context from 100 to 8000 keys once its
  // workgroups make about two trips each (batch 16, 2048 keys: 3660 -> 3739 tokens/s for the whole decode step;
  // batch 1, 8000 keys: 29.1 us with the row kernel, 32.1 with 9 wide splits per head, 27.0 with 16).  Splits per
  // head: two trips per workgroup, but no fewer workgroups than 288 (about one per CU: fewer leave CUs idle) and no
  // more than 512 (more splits mean more states to merge); the row kernel (TPPX_ATTN_WIDE=0) wants about two
  // workgroups per CU.  At most one split per trip and at most 32 (the merge holds every split's state in registers).
  const int wide_env = (int)env_int("TPPX_ATTN_WIDE", -1);
  const int64_t target_env = env_int("TPPX_ATTN_TARGET_WGS", 0);
  const bool wide = wide_env != 0;
  const int64_t heads = B * Nq;
  int64_t splits;
  if (target_env > 0 || !wide) {
    splits = ((target_env > 0 ? target_env : 512) + heads - 1) / heads;
  } else {
    const int64_t lo = (288 + heads - 1) / heads, hi = (512 + heads - 1) / heads;
    splits = ((Smax + ATTN_WIDE_KEYS - 1) / ATTN_WIDE_KEYS + 1) / 2;
    splits = splits < lo ? lo : splits > hi ? hi : splits;
  }
  const int64_t trip_keys = wide ? ATTN_WIDE_KEYS : 64;
  const int64_t max_by_len = (Smax + trip_keys - 1) / trip_keys;
  if (splits > max_by_len)
    splits = max_by_len;
  if (splits > 32)
    splits = 32;
  const int64_t need = B * Nq * splits * 130 * (int64_t)sizeof(float);
  if (splits > 1 && need > ws_bytes)
    splits = 1; // no room for partial results: one workgroup per head
  p.splits = (int)splits;
  p.part = (float*)ws;
  p.ticket0 = -1;
  if (splits > 1 && B * Nq <= ATTN_TICKETS && env_int("TPPX_ATTN_ONE_LAUNCH", 1) != 0) {
    // window of B * Nq arrival counters, handed out in rotation so that split launches in flight on different
    // streams do not share counters
    static std::mutex mu;
    static int cursor = 0;
    std::lock_guard<std::mutex> lock(mu);
    if (cursor + B * Nq > ATTN_TICKETS)
      cursor = 0;
    p.ticket0 = cursor;
    cursor += (int)(B * Nq);
  }
  const dim3 grid((unsigned)(B * Nq), (unsigned)splits);
  if (wide && rot)
    attn_decode_wide_kernel<true><<<grid, dim3(256), 0, stream>>>(p);
  else if (wide)
    attn_decode_wide_kernel<false><<<grid, dim3(256), 0, stream>>>(p);
  else if (rot)
    attn_decode_kernel<true><<<grid, dim3(256), 0, stream>>>(p);
  else
    attn_decode_kernel<false><<<grid, dim3(256), 0, stream>>>(p);
  int rc = check_hip(hipGetLastError(), who);
  if (rc && p.ticket0 >= 0) {
    // the refused launch leaves its counter window as it found it, but whoever gets the window next relies on zeros
    const int n = (int)(B * Nq);
    attn_clear_tickets_kernel<<<dim3((n + 255) / 256), dim3(256), 0, stream>>>(p.ticket0, n);
    (void)hipGetLastError();
  }
  if (rc || splits == 1 || p.ticket0 >= 0)
    return rc;
  attn_combine_kernel<<<dim3((unsigned)(B * Nq)), dim3(128), 0, stream>>>(p);
  return check_hip(hipGetLastError(), who);
}

// ---------------------------------------------------------------------------
// Attention for head sizes other than 128 (attn<T>, src/csrc/llm/attn.cpp:781-955, is generic in the head size; the
// kernels above are built for 128), H a multiple of 8 up to 256.  The single-query step runs on
// attn_generic_rows_kernel below, prompt passes on attn_prefill_hd_kernel above; this first, plain kernel serves
// both when those are switched off (TPPX_ATTN_GENERIC_ROWS=0, TPPX_ATTN_PREFILL_MFMA=0).  One wave per (sequence,
// query token, query head), four per workgroup, no barrier: 64 keys per trip,
// a lane takes the whole dot product of its key (16-byte loads along its row, the query as fp32 in wave-private
// LDS, read as broadcasts), online softmax over the trip with the probabilities rounded to bf16 before they multiply
// V and the normaliser summing the unrounded ones, then lanes turn to output dimensions (lane, lane + 64, ...) and
// walk the trip's value rows.  A plain kernel for the shapes the tuned ones do not take, not a tuned one.
// ---------------------------------------------------------------------------
struct AttnGenParams {
  const uint16_t* q;   // [B][S][Nq][H]
  const uint16_t* kc;  // [B][Nkv][Smax][H]
  const uint16_t* vc;
  const uint16_t* mask; // bf16 [B][mask_ld] additive, or null
  const int32_t* kv_len; // single-query step: device scalar, valid keys = *kv_len + kv_len_add; null: prompt pass
  int kv_len_add;
  uint16_t* out;       // [B][S][Nq][H]
  int B, S, Nq, Nkv, H, Smax, mask_ld, past; // prompt pass: query i sees keys 0 .. past + i
  float scale;
  int splits;          // single-query step (attn_generic_rows_kernel): workgroups per query, see there
  float* part;         // splits > 1: [query][split][2 + H] floats (running maximum, sum, unnormalised output)
};

__global__ void __launch_bounds__(256)
attn_generic_kernel(const AttnGenParams p) {
  __shared__ __align__(16) float q_s[4][256];
  __shared__ float p_s[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t qi = (int64_t)blockIdx.x * 4 + wave;
  if (qi >= (int64_t)p.B * p.S * p.Nq) // whole waves; nothing below synchronises across waves
    return;
  const int h = (int)(qi % p.Nq), sq = (int)((qi / p.Nq) % p.S), b = (int)(qi / ((int64_t)p.Nq * p.S));
  const int hk = h / (p.Nq / p.Nkv), H = p.H;
  int L = p.kv_len ? p.kv_len[0] + p.kv_len_add : p.past + sq + 1;
  L = max(min(L, p.Smax), 0);
  const uint16_t* qrow = p.q + qi * H;
  for (int d = lane; d < H; d += 64)
    q_s[wave][d] = bf16_bits_to_f32(qrow[d]);
  // the lanes of a wave hand values to one another through LDS: the LDS serves a wave's accesses in order; the
  // fence and the wave barrier keep the compiler from moving the reads above the writes
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  const uint16_t* kb = p.kc + ((int64_t)b * p.Nkv + hk) * (int64_t)p.Smax * H;
  const uint16_t* vb = p.vc + ((int64_t)b * p.Nkv + hk) * (int64_t)p.Smax * H;
  const uint16_t* mrow = p.mask ? p.mask + (int64_t)b * p.mask_ld : nullptr;
  float m = -3.0e38f, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int c0 = 0; c0 < L; c0 += 64) {
    const int key = c0 + lane;
    const uint16_t* krow = kb + (int64_t)min(key, L - 1) * H;
    float d = 0.f;
    for (int e = 0; e < H; e += 8) {
      const i32x4 kv = *reinterpret_cast<const i32x4*>(krow + e);
      const f32x4 qa = *reinterpret_cast<const f32x4*>(&q_s[wave][e]), qb = *reinterpret_cast<const f32x4*>(&q_s[wave][e + 4]);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const uint32_t w = (uint32_t)kv[j];
        const float q0 = j < 2 ? qa[2 * j] : qb[2 * j - 4], q1 = j < 2 ? qa[2 * j + 1] : qb[2 * j - 3];
        d = fmaf(bf16_bits_to_f32(w & 0xffffu), q0, d);
        d = fmaf(bf16_bits_to_f32(w >> 16), q1, d);
      }
    }
    d *= p.scale;
    if (mrow && key < p.mask_ld && key < L)
      d += bf16_bits_to_f32(mrow[key]);
    const float sc = key < L ? d : -3.0e38f;
    const float mn = fmaxf(m, wave_max(sc));
    const float alpha = __expf(m - mn); // 1 when the maximum stays
    m = mn;
    const float pr = key < L ? __expf(sc - m) : 0.f;
    l = l * alpha + wave_sum(pr);
#pragma unroll
    for (int i = 0; i < 4; i++)
      acc[i] *= alpha;
    __builtin_amdgcn_wave_barrier(); // (the previous trip's reads of p_s are done)
    p_s[wave][lane] = round_bf16(pr);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int nk = min(64, L - c0);
    for (int j = 0; j < nk; j++) {
      const float pj = p_s[wave][j];
      const uint16_t* vrow = vb + (int64_t)(c0 + j) * H;
#pragma unroll
      for (int i = 0; i < 4; i++)
        if (lane + 64 * i < H)
          acc[i] = fmaf(pj, bf16_bits_to_f32(vrow[lane + 64 * i]), acc[i]);
    }
  }
  uint16_t* orow = p.out + qi * H;
#pragma unroll
  for (int i = 0; i < 4; i++)
    if (lane + 64 * i < H)
      orow[lane + 64 * i] = (uint16_t)f32_to_bf16_bits(l > 0.f ? acc[i] / l : 0.f);
}

// The single-query step at those head sizes, laid out like attn_decode_kernel: G = 8, 16 or 32 lanes share a key
// (lane = key slot l / G, 16-byte chunk l % G; chunks past H / 8 idle), so a wave instruction reads 64 / G whole
// rows; NU instructions per wave and trip with the next trip requested ahead; every lane group keeps its own
// running (maximum, sum, 8 output dims per lane), merged at the end through LDS.  Grid (B * Nq, splits): split y
// takes the trips y, y + splits, ...; several splits leave their states for attn_generic_merge_kernel.
template <int G>
__global__ void __launch_bounds__(256)
attn_generic_rows_kernel(const AttnGenParams p) {
  constexpr int KPI = 64 / G;            // keys per wave instruction
  constexpr int NU = G == 8 ? 2 : 4;     // instructions per wave and trip
  constexpr int WK = NU * KPI;           // keys per wave and trip
  constexpr int TRIP = 4 * WK;           // keys per workgroup and trip
  constexpr int NG = 4 * KPI;            // lane groups per workgroup
  __shared__ float sm[NG], sl[NG];
  __shared__ float sacc[NG * G * 8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = lane / G, c = lane % G;
  const int H = p.H, C = H >> 3;
  const bool live = c < C;               // this lane's chunk exists
  const int cc = min(c, C - 1);
  const int bh = blockIdx.x, b = bh / p.Nq, hq = bh - b * p.Nq;
  const int hk = hq / (p.Nq / p.Nkv);
  const uint16_t* kb = p.kc + ((int64_t)b * p.Nkv + hk) * (int64_t)p.Smax * H + cc * 8;
  const uint16_t* vb = p.vc + ((int64_t)b * p.Nkv + hk) * (int64_t)p.Smax * H + cc * 8;
  i32x4 kw[NU], vw[NU], kn[NU], vn[NU];
  auto load_kv = [&](int base, i32x4 (&kd)[NU], i32x4 (&vd)[NU]) {
#pragma unroll
    for (int u = 0; u < NU; u++) {
      const int kk = min(base + u * KPI + grp, p.Smax - 1);
      kd[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(kb + (int64_t)kk * H));
      vd[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(vb + (int64_t)kk * H));
    }
  };
  load_kv(blockIdx.y * TRIP + wave * WK, kw, vw); // the first trip does not depend on the length (a device scalar)
  const int L = max(0, min(p.kv_len[0] + p.kv_len_add, p.Smax));
  const int trips = (L + TRIP - 1) / TRIP;
  float qf[8];
  unpack8(*reinterpret_cast<const uint4*>(p.q + (int64_t)bh * H + cc * 8), qf);
#pragma unroll
  for (int e = 0; e < 8; e++)
    qf[e] = live ? qf[e] * p.scale : 0.f;
  const uint16_t* mrow = p.mask ? p.mask + (int64_t)b * p.mask_ld : nullptr;
  float m = -3.0e38f, l = 0.f, acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++)
    acc[e] = 0.f;
  for (int t = blockIdx.y; t < trips; t += p.splits) {
    const int base = t * TRIP + wave * WK;
    load_kv(base + p.splits * TRIP, kn, vn); // unconditional (rows are clamped): a branch here would drain the queue
    float sc[NU];
    int key[NU];
#pragma unroll
    for (int u = 0; u < NU; u++) {
      key[u] = base + u * KPI + grp;
      float kf[8];
      unpack8(as_uint4(kw[u]), kf);
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++)
        d = fmaf(qf[e], kf[e], d);
      // sum over the G lanes of the key: DPP steps inside a row of 16, then the other half of a 32-lane group
      d += dpp_mov<0xB1>(d);
      d += dpp_mov<0x4E>(d);
      d += dpp_mov<0x141>(d);
      if (G >= 16)
        d += dpp_mov<0x140>(d);
      if (G == 32)
        d += __shfl_xor(d, 16);
      if (mrow && key[u] < p.mask_ld && key[u] < L)
        d += bf16_bits_to_f32(mrow[key[u]]);
      sc[u] = key[u] < L ? d : -3.0e38f;
    }
    if (t * TRIP + TRIP > L) { // the last trip only (wave-uniform): rows past the end may hold anything, NaN included
#pragma unroll
      for (int u = 0; u < NU; u++)
        if (key[u] >= L)
          vw[u] = i32x4{0, 0, 0, 0};
    }
    float mn = m;
#pragma unroll
    for (int u = 0; u < NU; u++)
      mn = fmaxf(mn, sc[u]);
    const float alpha = __expf(m - mn);
    l *= alpha;
#pragma unroll
    for (int e = 0; e < 8; e++)
      acc[e] *= alpha;
#pragma unroll
    for (int u = 0; u < NU; u++) {
      const float pr = key[u] < L ? __expf(sc[u] - mn) : 0.f;
      l += pr;
      const float pb = round_bf16(pr); // the probabilities that multiply V are bf16, the normaliser sums the unrounded
      float vf[8];
      unpack8(as_uint4(vw[u]), vf);
#pragma unroll
      for (int e = 0; e < 8; e++)
        acc[e] = fmaf(pb, vf[e], acc[e]);
    }
    m = mn;
#pragma unroll
    for (int u = 0; u < NU; u++) {
      kw[u] = kn[u];
      vw[u] = vn[u];
    }
  }
  // merge the lane groups of the workgroup
  const int gi = wave * KPI + grp;
  if (c == 0) {
    sm[gi] = m;
    sl[gi] = l;
  }
  if (live) {
#pragma unroll
    for (int e = 0; e < 8; e++)
      sacc[gi * (G * 8) + c * 8 + e] = acc[e];
  }
  __syncthreads();
  if (tid < H) {
    float M = -3.0e38f;
#pragma unroll
    for (int g = 0; g < NG; g++)
      M = fmaxf(M, sm[g]);
    float Ls = 0.f, o = 0.f;
#pragma unroll
    for (int g = 0; g < NG; g++) {
      const float w = __expf(sm[g] - M);
      Ls = fmaf(w, sl[g], Ls);
      o = fmaf(w, sacc[g * (G * 8) + tid], o);
    }
    if (p.splits == 1) {
      p.out[(int64_t)bh * H + tid] = (uint16_t)f32_to_bf16_bits(Ls > 0.f ? o / Ls : 0.f);
    } else {
      float* st = p.part + ((int64_t)bh * p.splits + blockIdx.y) * (int64_t)(H + 2);
      st[2 + tid] = o;
      if (tid == 0) {
        st[0] = M;
        st[1] = Ls;
      }
    }
  }
}

// one wave per query: the splits' (maximum, sum, output) states, in split order, become the normalised output
__global__ void __launch_bounds__(64)
attn_generic_merge_kernel(const AttnGenParams p) {
  const int lane = threadIdx.x;
  const int64_t qi = blockIdx.x;
  const int H = p.H;
  const float* st = p.part + qi * p.splits * (int64_t)(H + 2);
  float M = -3.0e38f;
  for (int i = 0; i < p.splits; i++)
    M = fmaxf(M, st[i * (H + 2)]);
  float Ls = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < p.splits; i++) {
    const float* si = st + i * (int64_t)(H + 2);
    const float w = __expf(si[0] - M); // a split without keys carries sum 0 and output 0
    Ls = fmaf(w, si[1], Ls);
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (lane + 64 * j < H)
        o[j] = fmaf(w, si[2 + lane + 64 * j], o[j]);
  }
  uint16_t* orow = p.out + qi * H;
#pragma unroll
  for (int j = 0; j < 4; j++)
    if (lane + 64 * j < H)
      orow[lane + 64 * j] = (uint16_t)f32_to_bf16_bits(Ls > 0.f ? o[j] / Ls : 0.f);
}

static int attn_generic_launch(const char* who, AttnGenParams& p, hipStream_t stream, void* ws = nullptr,
                               int64_t ws_bytes = 0) {
  TPPX_REQUIRE(p.H >= 8 && p.H <= 256 && p.H % 8 == 0, TPPX_EUNSUPPORTED,
               "%s: head size %d (128 on the tuned kernels, other multiples of 8 up to 256 on the plain one)", who, p.H);
  const int64_t queries = (int64_t)p.B * p.S * p.Nq;
  p.splits = 1;
  if (p.kv_len && p.S == 1 && env_int("TPPX_ATTN_GENERIC_ROWS", 1) != 0) {
    // Single-query steps: a workgroup per (query, split of the key range).  Up to 384 workgroups in all (measured at
    // 2048 keys: 16 heads of 256 59.9 -> 21.1 us with 24 splits, 64 queries 57.8 -> 27.6 us with 6, 256 queries
    // better unsplit), at least two trips each at the cache's capacity (the length itself is a device scalar: splits
    // whose trips lie past the keys leave empty states), at most 32; one split for caches under 512 keys (the merge
    // launch costs more than it saves) and when the caller's workspace cannot hold the states.
    const int G = p.H <= 64 ? 8 : p.H <= 128 ? 16 : 32;
    const int trip = G == 32 ? 32 : 64;
    int64_t want = env_int("TPPX_ATTN_GENERIC_SPLITS", 0);
    if (want <= 0)
      want = p.Smax < 512 ? 1 : 384 / queries;
    want = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, 32), ((int64_t)p.Smax + 2 * trip - 1) / (2 * trip)));
    if (want > 1 && ws && queries * want * (p.H + 2) * (int64_t)sizeof(float) <= ws_bytes) {
      p.splits = (int)want;
      p.part = (float*)ws;
    }
    TPPX_REQUIRE(queries < ((int64_t)1 << 31), TPPX_ESHAPE, "%s: problem too large", who);
    const dim3 grid((unsigned)queries, (unsigned)p.splits);
    if (G == 8)
      attn_generic_rows_kernel<8><<<grid, dim3(256), 0, stream>>>(p);
    else if (G == 16)
      attn_generic_rows_kernel<16><<<grid, dim3(256), 0, stream>>>(p);
    else
      attn_generic_rows_kernel<32><<<grid, dim3(256), 0, stream>>>(p);
    int rc = check_hip(hipGetLastError(), who);
    if (rc || p.splits == 1)
      return rc;
    attn_generic_merge_kernel<<<dim3((unsigned)queries), dim3(64), 0, stream>>>(p);
    return check_hip(hipGetLastError(), who);
  }
  const int64_t waves = queries;
  TPPX_REQUIRE(waves > 0 && (waves + 3) / 4 < ((int64_t)1 << 31), TPPX_ESHAPE, "%s: problem too large", who);
  attn_generic_kernel<<<dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, stream>>>(p);
  return check_hip(hipGetLastError(), who);
}

extern "C" int tppx_attn_decode(const void* q, const void* kcache, const void* vcache, const void* mask,
                                int64_t mask_ld, const void* kv_len_dev, int64_t kv_len_add, void* out, int64_t B, int64_t Nq,
                                int64_t Nkv, int64_t H, int64_t Smax, void* ws, int64_t ws_bytes,
                                tppx_stream_t stream) {
  const char* who = "tppx_attn_decode";
  TPPX_REQUIRE(q && kcache && vcache && kv_len_dev && out, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(q) && aligned16(kcache) && aligned16(vcache) && aligned16(out), TPPX_EINVAL,
               "%s: pointer not 16-byte aligned", who);
  TPPX_REQUIRE(B > 0 && Nq > 0 && Nkv > 0 && Nq % Nkv == 0 && Smax > 0 && B * Nq < (1 << 30), TPPX_ESHAPE,
               "%s: bad shape B=%ld Nq=%ld Nkv=%ld Smax=%ld", who, (long)B, (long)Nq, (long)Nkv, (long)Smax);
  TPPX_REQUIRE(ws_bytes >= 0 && (ws_bytes == 0 || ws), TPPX_EINVAL, "%s: workspace size given with a null workspace", who);
  if (H != 128) { // other head sizes: the plain kernel
    AttnGenParams g;
    memset(&g, 0, sizeof(g));
    g.q = (const uint16_t*)q; g.kc = (const uint16_t*)kcache; g.vc = (const uint16_t*)vcache; g.mask = (const uint16_t*)mask;
    g.kv_len = (const int32_t*)kv_len_dev; g.kv_len_add = (int)kv_len_add; g.out = (uint16_t*)out;
    g.B = (int)B; g.S = 1; g.Nq = (int)Nq; g.Nkv = (int)Nkv; g.H = (int)H; g.Smax = (int)Smax; g.mask_ld = (int)mask_ld;
    g.scale = 1.0f / sqrtf((float)H);
    return attn_generic_launch(who, g, (hipStream_t)stream, ws, ws_bytes);
  }
  AttnParams p;
  memset(&p, 0, sizeof(p));
  p.q = (const uint16_t*)q; p.kc = (const uint16_t*)kcache; p.vc = (const uint16_t*)vcache;
  p.mask = (const uint16_t*)mask; p.kv_len = (const int32_t*)kv_len_dev; p.kv_len_add = (int)kv_len_add; p.out = (uint16_t*)out;
  p.B = (int)B; p.Nq = (int)Nq; p.Nkv = (int)Nkv; p.Smax = (int)Smax; p.mask_ld = (int)mask_ld;
  p.scale = 1.0f / sqrtf((float)H);
  return attn_decode_launch(who, p, false, B, Nq, Smax, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int tppx_attn_decode_rotary(const void* q, const void* k, const void* v, const void* emb_pos,
                                       const void* pos, int64_t B_pos, int64_t MP, int64_t HR, void* kcache,
                                       void* vcache, const void* mask, int64_t mask_ld, const void* kv_len_dev,
                                       void* out, int64_t B, int64_t Nq, int64_t Nkv, int64_t H, int64_t Smax,
                                       void* ws, int64_t ws_bytes, tppx_stream_t stream) {
  const char* who = "tppx_attn_decode_rotary";
  TPPX_REQUIRE(q && k && v && pos && kcache && vcache && kv_len_dev && out, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(kcache) && aligned16(vcache) && aligned16(out) &&
                   (!emb_pos || aligned16(emb_pos)),
               TPPX_EINVAL, "%s: pointer not 16-byte aligned", who);
  TPPX_REQUIRE(H == 128 && (!emb_pos || HR == 128), TPPX_EUNSUPPORTED,
               "%s: head size %ld / rotary size %ld (only 128 with a full-width rotation is built)", who, (long)H, (long)HR);
  TPPX_REQUIRE(B > 0 && Nq > 0 && Nkv > 0 && Nq % Nkv == 0 && Smax > 0 && B * Nq < (1 << 30) && (B_pos == 1 || B_pos == B) &&
                   (!emb_pos || MP > 0),
               TPPX_ESHAPE, "%s: bad shape B=%ld Nq=%ld Nkv=%ld Smax=%ld B_pos=%ld MP=%ld", who, (long)B, (long)Nq,
               (long)Nkv, (long)Smax, (long)B_pos, (long)MP);
  TPPX_REQUIRE(ws_bytes >= 0 && (ws_bytes == 0 || ws), TPPX_EINVAL, "%s: workspace size given with a null workspace", who);
  AttnParams p;
  memset(&p, 0, sizeof(p));
  p.q = (const uint16_t*)q; p.kc = (const uint16_t*)kcache; p.vc = (const uint16_t*)vcache;
  p.mask = (const uint16_t*)mask; p.kv_len = (const int32_t*)kv_len_dev; p.kv_len_add = 1; p.out = (uint16_t*)out;
  p.B = (int)B; p.Nq = (int)Nq; p.Nkv = (int)Nkv; p.Smax = (int)Smax; p.mask_ld = (int)mask_ld;
  p.scale = 1.0f / sqrtf((float)H);
  p.k_new = (const uint16_t*)k; p.v_new = (const uint16_t*)v; p.emb = (const float*)emb_pos; p.pos = (const int64_t*)pos;
  p.MP = (int)MP; p.B_pos = (int)B_pos;
  return attn_decode_launch(who, p, true, B, Nq, Smax, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int tppx_attn_prefill(const void* q, const void* kcache, const void* vcache, const void* mask,
                                 int64_t mask_ld, int64_t past_len, void* out, int64_t B, int64_t S, int64_t Nq,
                                 int64_t Nkv, int64_t H, int64_t Smax, tppx_stream_t stream) {
  const char* who = "tppx_attn_prefill";
  TPPX_REQUIRE(q && kcache && vcache && out, TPPX_EINVAL, "%s: null pointer", who);
  TPPX_REQUIRE(aligned16(q) && aligned16(kcache) && aligned16(vcache) && aligned16(out), TPPX_EINVAL,
               "%s: pointer not 16-byte aligned", who);
  TPPX_REQUIRE(B > 0 && S > 0 && Nq > 0 && Nkv > 0 && Nq % Nkv == 0 && Smax > 0 && B * Nq < 65536 &&
                   S < ((int64_t)1 << 24) && Smax < ((int64_t)1 << 30),
               TPPX_ESHAPE, "%s: bad shape B=%ld S=%ld Nq=%ld Nkv=%ld Smax=%ld", who, (long)B, (long)S, (long)Nq,
               (long)Nkv, (long)Smax);
  TPPX_REQUIRE(past_len >= 0 && past_len + S <= Smax, TPPX_ESHAPE,
               "%s: %ld cached + %ld new keys exceed the cache capacity %ld", who, (long)past_len, (long)S, (long)Smax);
  TPPX_REQUIRE(!mask || mask_ld > 0, TPPX_EINVAL, "%s: mask given with mask_ld=%ld", who, (long)mask_ld);
  if (H != 128 && env_int("TPPX_ATTN_PREFILL_MFMA", 1) == 0) { // other head sizes on the plain kernel
    AttnGenParams g;
    memset(&g, 0, sizeof(g));
    g.q = (const uint16_t*)q; g.kc = (const uint16_t*)kcache; g.vc = (const uint16_t*)vcache; g.mask = (const uint16_t*)mask;
    g.out = (uint16_t*)out;
    g.B = (int)B; g.S = (int)S; g.Nq = (int)Nq; g.Nkv = (int)Nkv; g.H = (int)H; g.Smax = (int)Smax; g.mask_ld = (int)mask_ld;
    g.past = (int)past_len;
    g.scale = 1.0f / sqrtf((float)H);
    return attn_generic_launch(who, g, (hipStream_t)stream);
  }
  AttnPrefillParams p;
  memset(&p, 0, sizeof(p));
  p.q = (const uint16_t*)q; p.kc = (const uint16_t*)kcache; p.vc = (const uint16_t*)vcache;
  p.mask = (const uint16_t*)mask; p.out = (uint16_t*)out;
  p.B = (int)B; p.S = (int)S; p.Nq = (int)Nq; p.Nkv = (int)Nkv; p.Smax = (int)Smax; p.mask_ld = (int)mask_ld;
  p.past = (int)past_len;
  p.scale = 1.0f / sqrtf((float)H);
  p.H = (int)H;
  if (H != 128) { // other head sizes: the same kernel over a padded head size
    TPPX_REQUIRE(H >= 8 && H <= 256 && H % 8 == 0, TPPX_EUNSUPPORTED,
                 "%s: head size %ld (multiples of 8 up to 256)", who, (long)H);
    const int hd = H <= 64 ? 64 : H <= 128 ? 128 : 256;
    const long wgs2h = ((S + 127) / 128) * B * Nq;
    const bool two = hd != 256 && S > 64 && env_int("TPPX_ATTN_QG", wgs2h >= 512 ? 2 : 1) == 2;
    const size_t lds = (size_t)(64 * (hd + 8) + hd * AP_VP) * sizeof(uint16_t);
    const dim3 grid((unsigned)((S + (two ? 127 : 63)) / (two ? 128 : 64)), (unsigned)(B * Nq));
    hipError_t e = hipSuccess;
#define TPPX_AP_HD(QG_, HD_)                                                                                          \
  do {                                                                                                               \
    e = allow_dynamic_lds(reinterpret_cast<const void*>(attn_prefill_hd_kernel<QG_, HD_>), lds);                     \
    if (e == hipSuccess)                                                                                             \
      attn_prefill_hd_kernel<QG_, HD_><<<grid, dim3(256), lds, (hipStream_t)stream>>>(p);                            \
  } while (0)
    if (hd == 64 && two)
      TPPX_AP_HD(2, 64);
    else if (hd == 64)
      TPPX_AP_HD(1, 64);
    else if (hd == 128 && two)
      TPPX_AP_HD(2, 128);
    else if (hd == 128)
      TPPX_AP_HD(1, 128);
    else
      TPPX_AP_HD(1, 256);
#undef TPPX_AP_HD
    if (e != hipSuccess)
      return check_hip(e, who);
    return check_hip(hipGetLastError(), who);
  }
  // 32 queries per wave (QG = 2) halve the LDS reads per MFMA at 226 registers, still two waves per SIMD; they win
  // when the launch still has two workgroups per CU (S = 2048, 32 heads: 97 us against 117 us; 16 x 128 queries
  // behind 1024 cached keys: 69 against 96 us) and lose below that (S = 512, 32 heads: 22.5 against 17 us)
  const long wgs2 = ((S + 127) / 128) * B * Nq;
  const int qg = env_int("TPPX_ATTN_QG", wgs2 >= 512 ? 2 : 1);
  if (qg == 2 && S > 64)
    attn_prefill_kernel<2><<<dim3((unsigned)((S + 127) / 128), (unsigned)(B * Nq)), dim3(256), 0, (hipStream_t)stream>>>(p);
  else
    attn_prefill_kernel<1><<<dim3((unsigned)((S + 63) / 64), (unsigned)(B * Nq)), dim3(256), 0, (hipStream_t)stream>>>(p);
  return check_hip(hipGetLastError(), who);
}
