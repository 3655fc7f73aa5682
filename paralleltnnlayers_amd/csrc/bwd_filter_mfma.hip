// Backward-filter on the matrix cores in four launches (ranks up to 64 per pass,
// even channel counts).  Same reassociation of the reference's 8-deep sums
// (Cuda_kernels/cp4Conv2dBackwardFilter.cu:64-257) as the general path:
//   A = FC^T x,  B = FH *v A,  Cc = FW *h B,  G3 = FK^T dy,  G2, G1 = adjoint taps
//   dFK = dy . Cc^T   dFC = x . G1^T   dFW[j] = <G3, shift_j B>   dFH[i] = <G2, shift_i A>
//   1. contract_split_kernel: both channel -> rank contractions as exact fp32
//      products on the bf16 matrix cores (three-way split of both operands, six
//      MFMAs per 16-channel chunk); a wave owns one (image, 32-pixel block, 32-rank
//      tile) and streams x / dy through a register ring, the factor tile sits
//      pre-split in LDS.  contract_mfma_kernel (plain fp32 MFMA) takes the channel
//      counts that are not multiples of 16.
//   2. taps: B, Cc, G2, G1 and the tap-gradient partials, one wave per (image, rank)
//      plane - taps_wave_kernel (planes up to 256 pixels, wave-private LDS) or
//      taps_column_kernel (lane = column, rows in registers); B and G2 never leave
//      the compute unit.  taps_plane_kernel / taps_kernel for the other filter shapes.
//   3. grad_split_kernel: dF[d,r] = sum_{n,p} act[n,d,p] Z[n,r,p] as split products,
//      split over images (and pixel ranges) across workgroups, the Z tile split once
//      per 32-pixel chunk into double-buffered B fragments in LDS.  grad_gemm_kernel
//      (fp32 MFMA) where rows cannot move as 16-byte vectors.
//   4. reduce4_kernel: fixed-order sum of the per-workgroup partials (bit-reproducible).
// The library's choice for large problems and for shapes the three-launch variant
// (bwd_filter_fused.hip) does not take; also the strided layer's pass and the
// 3-factor op's (depthwise-filter tap step).
#include <cstdint>
#include <cstdlib>

#include "cp4_internal.h"
#ifdef CP4_DEBUG_PHASES
#include "cp4_debug.h"
#endif
#include "split_bf16.h"

// Compiled twice more with CP4_BWF_IO16: x and dy are then 16-bit in memory (factors,
// intermediates and gradients stay fp32).  Only the split-bf16 kernels exist in
// those builds (contract_split_kernel, grad_split_kernel).  CP4_BWF_IO16 == 1,
// bfloat16: an activation is its own high part, so neither kernel splits its
// activations and both run three MFMAs per product instead of six; entry points
// bwd_filter_mfma_io16_*.  CP4_BWF_IO16 == 2, IEEE half: 11 significand bits are two
// bf16 parts (8 + 3), five MFMAs per product; entry points bwd_filter_mfma_iof16_*.
#if defined(CP4_BWF_IO16) && CP4_BWF_IO16 == 2
#define bwd_filter_mfma_supported bwd_filter_mfma_iof16_supported
#define bwd_filter_mfma_workspace_bytes bwd_filter_mfma_iof16_workspace_bytes
#define bwd_filter_mfma_launch bwd_filter_mfma_iof16_launch
#define CP4_BWF_HALF 1
#elif defined(CP4_BWF_IO16)
#define bwd_filter_mfma_supported bwd_filter_mfma_io16_supported
#define bwd_filter_mfma_workspace_bytes bwd_filter_mfma_io16_workspace_bytes
#define bwd_filter_mfma_launch bwd_filter_mfma_io16_launch
#endif

namespace cp4 {
namespace {

#ifdef CP4_BWF_HALF
using act_t = unsigned short;      // IEEE half bits
[[maybe_unused]] __device__ __forceinline__ float act_to_f32(act_t v) {
  return (float)__builtin_bit_cast(_Float16, v);
}
// Exact split of 8 half-precision values (widened to fp32) into two bf16 parts.
[[maybe_unused]] __device__ __forceinline__ void split8_half(const float (&v)[8], split::u32x4& h,
                                                             split::u32x4& m) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const float a = v[2 * d], b = v[2 * d + 1];
    h[d] = split::pack_hi16(a, b);
    m[d] = split::pack_hi16(a - split::trunc_bf16(a), b - split::trunc_bf16(b));
  }
}
#elif defined(CP4_BWF_IO16)
using act_t = unsigned short;      // bfloat16 bits
[[maybe_unused]] __device__ __forceinline__ float act_to_f32(act_t v) {
  return __uint_as_float((unsigned)v << 16);
}
#else
using act_t = float;
[[maybe_unused]] __device__ __forceinline__ float act_to_f32(act_t v) { return v; }
#endif

using split::f32x16;

[[maybe_unused]] __device__ __forceinline__ f32x16 mfma32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

#ifdef CP4_DEBUG_PHASES
// Debug builds: wall-clock stamps per (kernel slot, workgroup, wave) into a caller's buffer.
#define BSTAMP(dbg, slot, wg, nw, i)                                                          \
  if ((dbg) && (threadIdx.x & 63) == 0)                                                       \
    (dbg)[(((size_t)(slot) * 4096 + (wg)) * (nw) + (threadIdx.x >> 6)) * 8 + (i)] = wall_clock64();
#else
#define BSTAMP(dbg, slot, wg, nw, i)
#endif
constexpr int kCT = 256;   // gradient-GEMM workgroup: 4 waves
[[maybe_unused]] constexpr int kCW = 256;   // contraction workgroup: 4 waves (one per SIMD) sharing one 32-rank factor tile
[[maybe_unused]] constexpr int kPF = 8;     // channel pairs per prefetch chunk in the contraction
[[maybe_unused]] constexpr int kSplitSlice = 768;   // channels per launch of the split contraction beyond its fragment tile
[[maybe_unused]] constexpr int kContractSlice = 1024;   // channels of the fp32 contraction's factor tile in LDS at a time

// ---- 1. Z[n,r,p] = sum_c F[c,r] src[n,c,p] ---------------------------------
struct ContractArgs {
  const act_t* src[2];   // x, dy
  const float* F[2];     // FC, FK
  float* Z[2];           // A, G3
  int Cin[2];
  int ldc[2];            // split kernel: channels of an image in memory when Cin is a slice of them (0: Cin)
  int N, R, RP, HW, npb, items;   // items per contraction and rank tile = N * npb
  int ks;   // split kernel: waves per item, each contracting 1/ks of the channels (1, 2 or 4)
  long long* dbg;
};

#ifndef CP4_BWF_IO16
__global__ __launch_bounds__(kCW) void contract_mfma_kernel(ContractArgs a) {
  extern __shared__ float Fs[];   // [slice of Cin][32]: the 32-rank tile mb of F, zero-padded
  const int which = blockIdx.y, mb = blockIdx.z;
  const int Cin = a.Cin[which], R = a.R, HW = a.HW;
  constexpr int RP = 32;
  const float* F = a.F[which];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  const int item = blockIdx.x * (kCW / 64) + wave;   // (image, 64-pixel block)
  const bool active = item < a.items;                 // (idle waves still meet the barriers)
  const int pb = active ? item % a.npb : 0, n = active ? item / a.npb : 0;
  const int p = pb * 64 + 2 * l32;
  const bool valid = active && p < HW;
  const int pc = valid ? p : HW - 2;
  const float* fp = Fs + hi * RP + l32;
  f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
  // the factor tile goes through LDS a slice of kContractSlice channels at a time
  for (int c0 = 0; c0 < Cin; c0 += kContractSlice) {
    const int cs = Cin - c0 < kContractSlice ? Cin - c0 : kContractSlice;
    if (c0) __syncthreads();                          // every wave is done with the last slice
    for (int i0 = tid; i0 < cs * 32; i0 += kCW * 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int i = i0 + u * kCW, c = c0 + (i >> 5), r = 32 * mb + (i & 31);
        v[u] = (i < cs * 32 && r < R) ? F[(size_t)c * R + r] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u)
        if (i0 + u * kCW < cs * 32) Fs[i0 + u * kCW] = v[u];
    }
    __syncthreads();
    if (!active) continue;
    const float* xp = a.src[which] + ((size_t)n * Cin + c0 + hi) * HW + pc;
    const int nsteps = cs >> 1, nchunks = nsteps / kPF;
    float2 xb0[kPF], xb1[kPF];
    auto load = [&](float2 (&xb)[kPF], int ch) {
#pragma unroll
      for (int s = 0; s < kPF; ++s)
        xb[s] = *reinterpret_cast<const float2*>(xp + (size_t)(2 * (ch * kPF + s)) * HW);
    };
    auto compute = [&](const float2 (&xb)[kPF], int ch) {
#pragma unroll
      for (int s = 0; s < kPF; ++s) {
        const float f = fp[(ch * kPF + s) * 2 * RP];
        acc0 = mfma32(f, xb[s].x, acc0);
        acc1 = mfma32(f, xb[s].y, acc1);
      }
    };
    if (nchunks > 0) load(xb0, 0);
    for (int ch = 0; ch < nchunks; ch += 2) {
      if (ch + 1 < nchunks) load(xb1, ch + 1);
      compute(xb0, ch);
      if (ch + 1 < nchunks) {
        if (ch + 2 < nchunks) load(xb0, ch + 2);
        compute(xb1, ch + 1);
      }
    }
    for (int st = nchunks * kPF; st < nsteps; ++st) {
      const float2 xv = *reinterpret_cast<const float2*>(xp + (size_t)(2 * st) * HW);
      const float f = fp[st * 2 * RP];
      acc0 = mfma32(f, xv.x, acc0);
      acc1 = mfma32(f, xv.y, acc1);
    }
  }
  if (valid) {
    float* zn = a.Z[which] + (size_t)n * R * HW + p;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int r = 32 * mb + 8 * (v >> 2) + 4 * hi + (v & 3);
      if (r < R) {
        float2 o;
        o.x = acc0[v];
        o.y = acc1[v];
        *reinterpret_cast<float2*>(zn + (size_t)r * HW) = o;
      }
    }
  }
}

#endif  // !CP4_BWF_IO16

// ---- 1'. the same contraction as exact fp32 products on the bf16 matrix cores
// (channel counts that are multiples of 16).  A workgroup of 8 waves shares the
// 32-rank factor tile as pre-split MFMA A fragments in LDS
// ([16-channel chunk][part][half][rank] x 16 B); a wave owns one (image,
// 32-pixel block): it streams x / dy through a register ring as the B operand,
// splits each 16-channel chunk and issues six bf16 MFMAs for it - 2.7x less
// matrix time than the fp32 MFMA and twice as many waves to hide latency with.
// When there are few items (small planes, small batches) ks = 2 or 4 adjacent
// waves share an item, each contracting 1/ks of the channels - shorter dependent
// load chains and ks times the waves - and add their partial sums through LDS
// in fixed order.
constexpr int kSplitRing = 4;
constexpr long kKsWaves = 1024;   // channel splits only while the grid stays below this many waves
constexpr int kSW = 512;    // 8 waves share one factor tile: one fill per workgroup
__global__ __launch_bounds__(kSW) void contract_split_kernel(ContractArgs a) {
  using namespace split;
  extern __shared__ float Fs[];
  unsigned char* Fb = reinterpret_cast<unsigned char*>(Fs);
  const int which = blockIdx.y, mb = blockIdx.z;
  const int Cin = a.Cin[which], R = a.R, HW = a.HW;
  const float* F = a.F[which];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  // This wave's item; waves past the end keep a valid (clamped) item for their
  // loads and skip the store, so that every wave reaches the barrier.
  const int ks = a.ks;
  [[maybe_unused]] const int dwg = (blockIdx.z * 2 + blockIdx.y) * gridDim.x + blockIdx.x;
  BSTAMP(a.dbg, 0, dwg, 8, 0)
  const int slot = blockIdx.x * (kSW / 64) + wave;        // (item, channel split)
  const int item_raw = slot / ks, part = slot - item_raw * ks;   // item = (image, 32-pixel block)
  const bool has_item = item_raw < a.items;
  const int item = has_item ? item_raw : a.items - 1;
  const int pb = item % a.npb, n = item / a.npb;
  const int p = pb * 32 + l32;
  const bool valid = has_item && p < HW;
  const int pc = p < HW ? p : HW - 1;
  // lane's channel 16*chunk + 8*hi + e
  const int nch = (Cin >> 4) / ks, c0 = part * nch;     // this wave's chunks c0 .. c0 + nch - 1
  const act_t* xp = a.src[which] +
                    ((size_t)n * (a.ldc[which] ? a.ldc[which] : Cin) + 16 * c0 + 8 * hi) * HW + pc;
#ifdef CP4_BWF_IO16
  using ring_t = unsigned;     // raw 16-bit values, zero-extended
#else
  using ring_t = float;
#endif
  ring_t xb[kSplitRing][8];
  auto ld_chunk = [&](ring_t (&dst)[8], int ch) {
    ch = ch < nch ? ch : nch - 1;                     // clamped, not branched
    const act_t* base = xp + (size_t)(16 * ch) * HW;
#pragma unroll
    for (int e = 0; e < 8; ++e) dst[e] = base[(size_t)e * HW];
  };
  // the first activation chunks are requested before the factor tile is built,
  // so their HBM latency runs under the fill
#pragma unroll
  for (int u = 0; u < kSplitRing; ++u) ld_chunk(xb[u], u);
  // two (channel octet, rank) entries per thread and round, their sixteen factor
  // loads issued together
  const int nfill = (Cin >> 3) * 32, fr = 32 * mb + (tid & 31);
  for (int it = tid; it < nfill; it += 2 * kSW) {
    float v[2][8];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int o = min(it + t * kSW, nfill - 1) >> 5;       // channel octet (clamped)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[t][e] = fr < R ? F[(size_t)(8 * o + e) * R + fr] : 0.f;
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (it + t * kSW >= nfill) break;
      const int o = (it + t * kSW) >> 5;
      u32x4 h, m, l;
      split8(v[t], h, m, l);
      u32x4* dst =
          reinterpret_cast<u32x4*>(Fb + ((size_t)(o >> 1) * 6 + (o & 1)) * 512 + (tid & 31) * 16);
      dst[0] = h;          // part stride: 2 planes of 512 B
      dst[64] = m;
      dst[128] = l;
    }
  }
  BSTAMP(a.dbg, 0, dwg, 8, 1)
  __syncthreads();
  BSTAMP(a.dbg, 0, dwg, 8, 2)
  const u32x4* fbase = reinterpret_cast<const u32x4*>(Fb + hi * 512 + l32 * 16);
  // Software pipeline: while the six MFMAs of chunk c run (two accumulators, so
  // they do not wait for each other), the vector ALU splits chunk c+1.
  f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
  u32x4 xh, xm, xl;
#ifdef CP4_BWF_HALF
  // half-precision activations: widened, then two bf16 parts
  auto pack8 = [](const ring_t (&v)[8], u32x4& h, u32x4& m) {
    float w[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = act_to_f32((act_t)v[e]);
    split8_half(w, h, m);
  };
  pack8(xb[0], xh, xm);
  xl = xh;                      // unused
#elif defined(CP4_BWF_IO16)
  // bfloat16 activations: the chunk's B operand is the packed bits themselves
  auto pack8 = [](const ring_t (&v)[8], u32x4& h, u32x4&) {
#pragma unroll
    for (int d = 0; d < 4; ++d) h[d] = v[2 * d] | (v[2 * d + 1] << 16);
  };
  pack8(xb[0], xh, xm);
  xm = xl = xh;                 // unused
#else
  split8(xb[0], xh, xm, xl);
#endif
  BSTAMP(a.dbg, 0, dwg, 8, 5)
  ld_chunk(xb[0], kSplitRing);
  for (int ch = 0; ch < nch; ch += kSplitRing) {
#pragma unroll
    for (int u = 0; u < kSplitRing; ++u) {
      const int c = ch + u;                           // chunk whose parts are in xh/xm/xl
      u32x4 nh = xh, nm = xm, nl = xl;
      if (c < nch) {
        const u32x4* fp = fbase + (size_t)(c0 + c) * (6 * 32);
        const u32x4 fh = fp[0], fm = fp[64], fl = fp[128];
        // one MFMA, then a quarter of the next chunk's split, pinned in this order
        ring_t (&nx)[8] = xb[(u + 1) % kSplitRing];
#ifdef CP4_BWF_HALF
        acc0 = mfma16(fl, xh, acc0);
        acc1 = mfma16(fm, xm, acc1);
        acc0 = mfma16(fm, xh, acc0);
        acc1 = mfma16(fh, xm, acc1);
        acc0 = mfma16(fh, xh, acc0);
        pack8(nx, nh, nm);
        ld_chunk(nx, c + 1 + kSplitRing);             // refill the slot just split
#elif defined(CP4_BWF_IO16)
        acc0 = mfma16(fl, xh, acc0);
        acc1 = mfma16(fm, xh, acc1);
        acc0 = mfma16(fh, xh, acc0);
        pack8(nx, nh, nm);
        ld_chunk(nx, c + 1 + kSplitRing);             // refill the slot just packed
#else
        auto piece = [&](int d) {
          const float x0 = nx[2 * d], x1 = nx[2 * d + 1];
          nh[d] = pack_hi16(x0, x1);
          const float r0 = x0 - trunc_bf16(x0), r1 = x1 - trunc_bf16(x1);
          nm[d] = pack_hi16(r0, r1);
          nl[d] = pack_hi16(r0 - trunc_bf16(r0), r1 - trunc_bf16(r1));
        };
        acc0 = mfma16(fl, xh, acc0);
        piece(0);
        __builtin_amdgcn_sched_barrier(0);
        acc1 = mfma16(fm, xm, acc1);
        piece(1);
        __builtin_amdgcn_sched_barrier(0);
        acc0 = mfma16(fh, xl, acc0);
        piece(2);
        __builtin_amdgcn_sched_barrier(0);
        acc1 = mfma16(fm, xh, acc1);
        piece(3);
        __builtin_amdgcn_sched_barrier(0);
        acc0 = mfma16(fh, xm, acc0);
        acc1 = mfma16(fh, xh, acc1);
        ld_chunk(nx, c + 1 + kSplitRing);             // refill the slot just split
#endif
      }
      xh = nh;
      xm = nm;
      xl = nl;
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  f32x16 acc = acc0 + acc1;
  BSTAMP(a.dbg, 0, dwg, 8, 3)
  float* zn = a.Z[which] + (size_t)n * R * HW + p;
  if (ks == 1) {
    if (valid) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = 32 * mb + 8 * (v >> 2) + 4 * hi + (v & 3);
        if (r < R) zn[(size_t)r * HW] = acc[v];
      }
    }
    BSTAMP(a.dbg, 0, dwg, 8, 4)
    return;
  }
  // ks waves hold partial sums of one item: exchange through LDS (over the
  // factor tile, which nobody reads any more) and let wave `part` add and store
  // rows v = part, part + ks, ... in the fixed order of the splits.
  __syncthreads();
  float* red = Fs;                                   // [wave][v][lane]
#pragma unroll
  for (int v = 0; v < 16; ++v) red[(wave * 16 + v) * 64 + lane] = acc[v];
  __syncthreads();
  const int w0 = wave - part;                        // first wave of this item
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    if ((v & (ks - 1)) != part) continue;            // wave-uniform
    float sum = 0.f;
    for (int q = 0; q < ks; ++q) sum += red[((w0 + q) * 16 + v) * 64 + lane];
    const int r = 32 * mb + 8 * (v >> 2) + 4 * hi + (v & 3);
    if (valid && r < R) zn[(size_t)r * HW] = sum;
  }
}

// ---- 2. taps: B, Cc from A; G2, G1 from G3 ----------------------------------
__global__ __launch_bounds__(256) void taps_kernel(const float* __restrict__ A,
                                                   const float* __restrict__ G3,
                                                   const float* __restrict__ FH,
                                                   const float* __restrict__ FW,
                                                   float* __restrict__ B, float* __restrict__ Cc,
                                                   float* __restrict__ G2, float* __restrict__ G1,
                                                   size_t total, int R, int H, int W, int Y,
                                                   int X, int P) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int w = idx % W, h = (idx / W) % H;
  const size_t plane = idx / ((size_t)W * H);
  const int r = plane % R;
  const float* ap = A + plane * (size_t)H * W;
  const float* gp = G3 + plane * (size_t)H * W;
  float b = 0.f, cc = 0.f, g2 = 0.f, g1 = 0.f;
  for (int i = 0; i < Y; ++i) {
    const float fh = FH[i * R + r];
    const int hf = h + i - P, hb = h - i + P;     // forward / adjoint row
    if (hf >= 0 && hf < H) {
      b += fh * ap[hf * W + w];
      float s = 0.f;
      for (int j = 0; j < X; ++j) {
        const int ww = w + j - P;
        if (ww >= 0 && ww < W) s += FW[j * R + r] * ap[hf * W + ww];
      }
      cc += fh * s;
    }
    if (hb >= 0 && hb < H) {
      float s = 0.f;
      for (int j = 0; j < X; ++j) {
        const int ww = w - j + P;
        if (ww >= 0 && ww < W) s += FW[j * R + r] * gp[hb * W + ww];
      }
      g1 += fh * s;
    }
  }
  for (int j = 0; j < X; ++j) {
    const int ww = w - j + P;
    if (ww >= 0 && ww < W) g2 += FW[j * R + r] * gp[h * W + ww];
  }
  B[idx] = b;
  Cc[idx] = cc;
  G2[idx] = g2;
  G1[idx] = g1;
}

// Same taps with one workgroup per (image, rank) plane held in LDS, which also
// yields the plane's tap-gradient partials: partH[n][i][r] = <G2, shift_i A>,
// partW[n][j][r] = <G3, shift_j B>.  Tap weights are workgroup-uniform.
__device__ __forceinline__ float block_sum256(float v, float* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

__global__ __launch_bounds__(256) void taps_plane_kernel(
    const float* __restrict__ A, const float* __restrict__ G3, const float* __restrict__ FH,
    const float* __restrict__ FW, float* __restrict__ B, float* __restrict__ Cc,
    float* __restrict__ G2, float* __restrict__ G1, float* __restrict__ partH,
    float* __restrict__ partW, int R, int H, int W, int Y, int X, int P) {
  extern __shared__ float pl[];
  const int HW = H * W;
  float *sA = pl, *sG = pl + HW, *sB = pl + 2 * HW, *sG2 = pl + 3 * HW;
  const int plane = blockIdx.x, r = plane % R, n = plane / R;
  const size_t base = (size_t)plane * HW;
  float* red = pl + 4 * HW;                       // [Y + X][4] wave partials
  float* fh = red + 4 * (Y + X);                  // this rank's tap weights, read once
  float* fw = fh + Y;
  for (int p = threadIdx.x; p < HW; p += 256) {
    sA[p] = A[base + p];
    sG[p] = G3[base + p];
  }
  if ((int)threadIdx.x < Y) fh[threadIdx.x] = FH[threadIdx.x * R + r];
  else if ((int)threadIdx.x < Y + X) fw[threadIdx.x - Y] = FW[(threadIdx.x - Y) * R + r];
  __syncthreads();
  for (int p = threadIdx.x; p < HW; p += 256) {
    const int h = p / W, w = p - h * W;
    float b = 0.f, g2 = 0.f;
    for (int i = 0; i < Y; ++i) {
      const int hh = h + i - P;
      if (hh >= 0 && hh < H) b += fh[i] * sA[hh * W + w];
    }
    for (int j = 0; j < X; ++j) {
      const int ww = w - j + P;
      if (ww >= 0 && ww < W) g2 += fw[j] * sG[h * W + ww];
    }
    sB[p] = b;
    sG2[p] = g2;
    B[base + p] = b;
    G2[base + p] = g2;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < HW; p += 256) {
    const int h = p / W, w = p - h * W;
    float cc = 0.f, g1 = 0.f;
    for (int j = 0; j < X; ++j) {
      const int ww = w + j - P;
      if (ww >= 0 && ww < W) cc += fw[j] * sB[h * W + ww];
    }
    for (int i = 0; i < Y; ++i) {
      const int hh = h - i + P;
      if (hh >= 0 && hh < H) g1 += fh[i] * sG2[hh * W + w];
    }
    Cc[base + p] = cc;
    G1[base + p] = g1;
  }
  // tap gradients of this plane: wave sums to LDS, one barrier, then a fixed-order
  // sum of the four wave partials per tap
  for (int t = 0; t < Y + X; ++t) {
    const bool vertical = t < Y;
    const int o = (vertical ? t : t - Y) - P;
    float acc = 0.f;
    for (int p = threadIdx.x; p < HW; p += 256) {
      const int h = p / W, w = p - h * W;
      const int hh = vertical ? h + o : h, ww = vertical ? w : w + o;
      if (hh >= 0 && hh < H && ww >= 0 && ww < W)
        acc += vertical ? sG2[p] * sA[hh * W + ww] : sG[p] * sB[hh * W + ww];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if ((threadIdx.x & 63) == 0) red[t * 4 + (threadIdx.x >> 6)] = acc;
  }
  __syncthreads();
  if ((int)threadIdx.x < Y + X) {
    const int t = threadIdx.x;
    const float tot = red[t * 4] + red[t * 4 + 1] + red[t * 4 + 2] + red[t * 4 + 3];
    if (t < Y) partH[((size_t)n * Y + t) * R + r] = tot;
    else partW[((size_t)n * X + (t - Y)) * R + r] = tot;
  }
}

// The 3-factor CP op's tap step (test/layers.py:265-282: a depthwise Y x X filter
// K1 [Y,X,R] between the two pointwise factors): one workgroup per (image, rank)
// plane in LDS, Cc = K1 (*) A, G1 = the adjoint taps of G3, and the plane's
// Y*X tap-gradient partials part[n][i*X+j][r] = <G3, shift_(i,j) A>.
__global__ __launch_bounds__(256) void taps2d_plane_kernel(
    const float* __restrict__ A, const float* __restrict__ G3, const float* __restrict__ K1,
    float* __restrict__ Cc, float* __restrict__ G1, float* __restrict__ part, int R, int H, int W,
    int Y, int X, int P) {
  extern __shared__ float pl[];
  const int HW = H * W, YX = Y * X;
  float *sA = pl, *sG = pl + HW;
  float* red = pl + 2 * HW;                       // [Y*X][4] wave partials
  float* wk = red + 4 * YX;                       // this rank's filter
  const int plane = blockIdx.x, r = plane % R, n = plane / R;
  const size_t base = (size_t)plane * HW;
  for (int p = threadIdx.x; p < HW; p += 256) {
    sA[p] = A[base + p];
    sG[p] = G3[base + p];
  }
  for (int t = threadIdx.x; t < YX; t += 256) wk[t] = K1[(size_t)t * R + r];
  __syncthreads();
  for (int p = threadIdx.x; p < HW; p += 256) {
    const int h = p / W, w = p - h * W;
    float cc = 0.f, g1 = 0.f;
    for (int i = 0; i < Y; ++i)
      for (int j = 0; j < X; ++j) {
        const float k = wk[i * X + j];
        const int hf = h + i - P, wf = w + j - P, hb = h - i + P, wb = w - j + P;
        if (hf >= 0 && hf < H && wf >= 0 && wf < W) cc += k * sA[hf * W + wf];
        if (hb >= 0 && hb < H && wb >= 0 && wb < W) g1 += k * sG[hb * W + wb];
      }
    Cc[base + p] = cc;
    G1[base + p] = g1;
  }
  for (int t = 0; t < YX; ++t) {
    const int oi = t / X - P, oj = t % X - P;
    float acc = 0.f;
    for (int p = threadIdx.x; p < HW; p += 256) {
      const int h = p / W, w = p - h * W, hh = h + oi, ww = w + oj;
      if (hh >= 0 && hh < H && ww >= 0 && ww < W) acc += sG[p] * sA[hh * W + ww];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if ((threadIdx.x & 63) == 0) red[t * 4 + (threadIdx.x >> 6)] = acc;
  }
  __syncthreads();
  for (int t = threadIdx.x; t < YX; t += 256)
    part[((size_t)n * YX + t) * R + r] = ((red[t * 4] + red[t * 4 + 1]) + red[t * 4 + 2]) + red[t * 4 + 3];
}

// Sum of v over the 64 lanes, valid in lane 63: a shift-and-add scan inside each
// row of 16 lanes, then the row totals passed on to the following rows, all as
// data-parallel-primitive moves (no LDS traffic).  Lanes a move does not reach
// read 0.
template <int CTRL, int ROW_MASK, bool BOUND>
__device__ __forceinline__ float dpp_move(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL,
                                                               ROW_MASK, 0xf, BOUND));
}
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v += dpp_move<0x111, 0xf, true>(v);    // row_shr:1
  v += dpp_move<0x112, 0xf, true>(v);    // row_shr:2
  v += dpp_move<0x114, 0xf, true>(v);    // row_shr:4
  v += dpp_move<0x118, 0xf, true>(v);    // row_shr:8: lane 15 of a row holds the row's sum
  v += dpp_move<0x142, 0xa, false>(v);   // row_bcast:15 into rows 1 and 3
  v += dpp_move<0x143, 0xc, false>(v);   // row_bcast:31 into rows 2 and 3
  return v;
}

// ---- 2'. the same for small planes: one WAVE per (image, rank) plane -------
// A plane of at most 256 pixels fits one wave with PP pixels per lane; its four
// intermediate planes live in a wave-private LDS slice, so there is no
// workgroup barrier, no idle thread and 4 planes per workgroup.  B and G2 stay
// on chip: only Cc, G1 and the tap-gradient partials leave the CU.
// The LDS planes carry a zero border of Q = max(P, FS-1-P) cells on every side,
// so that every tap is an unconditional read at a fixed offset from the pixel's
// cell: no bounds arithmetic in the tap loops.
template <int FS, int PP>
__global__ __launch_bounds__(256) void taps_wave_kernel(
    const float* __restrict__ A, const float* __restrict__ G3, const float* __restrict__ FH,
    const float* __restrict__ FW, float* __restrict__ Cc, float* __restrict__ G1,
    float* __restrict__ partH, float* __restrict__ partW, int R, int H, int W, int P, int Q,
    unsigned wmagic, int nplanes) {
  extern __shared__ __attribute__((aligned(16))) float pl[];
  const int HW = H * W, Wp = W + 2 * Q, cells = (H + 2 * Q) * Wp;   // cells: multiple of 4 (host)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int plane = blockIdx.x * 4 + wave;
  if (plane >= nplanes) return;                   // whole wave; no workgroup barrier below
  const int r = plane % R, n = plane / R;
  float* sA = pl + (size_t)wave * 4 * cells;
  float *sG = sA + cells, *sB = sA + 2 * cells, *sG2 = sA + 3 * cells;
  const size_t base = (size_t)plane * HW;
  // the plane's values are requested first, the LDS clear runs under their latency
  float a[PP], g[PP];
#pragma unroll
  for (int k = 0; k < PP; ++k) {
    const int p = min(lane + 64 * k, HW - 1);     // only the last k can pass the end
    a[k] = A[base + p];
    g[k] = G3[base + p];
  }
  float fh[FS], fw[FS];
#pragma unroll
  for (int i = 0; i < FS; ++i) {
    fh[i] = FH[i * R + r];
    fw[i] = FW[i * R + r];
  }
  for (int q = lane; q < cells; q += 64)          // 4 planes x cells floats = cells float4
    reinterpret_cast<float4*>(sA)[q] = make_float4(0.f, 0.f, 0.f, 0.f);
  // cell of pixel k in a padded plane; lanes past the plane's end take pixel 0's
  // cell: they recompute and rewrite that pixel's values and add nothing to the sums
  int c[PP];
  bool ok[PP];
#pragma unroll
  for (int k = 0; k < PP; ++k) {
    const int p = lane + 64 * k;
    ok[k] = k < PP - 1 || p < HW;
    const int pc = ok[k] ? p : 0;
    const int h = (int)__umulhi((unsigned)pc, wmagic), w = pc - h * W;
    c[k] = (h + Q) * Wp + w + Q;
    if (!ok[k]) g[k] = 0.f;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int k = 0; k < PP; ++k)
    if (ok[k]) {
      sA[c[k]] = a[k];
      sG[c[k]] = g[k];
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  float av[PP][FS], g2[PP];
#pragma unroll
  for (int k = 0; k < PP; ++k) {
    float b = 0.f, v = 0.f;
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      av[k][i] = sA[c[k] + (i - P) * Wp];         // A one row per tap below / above
      b += fh[i] * av[k][i];
      v += fw[i] * sG[c[k] + (P - i)];
    }
    if (ok[k]) {
      sB[c[k]] = b;
      sG2[c[k]] = v;
    }
    g2[k] = ok[k] ? v : 0.f;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  float accH[FS], accW[FS];
#pragma unroll
  for (int i = 0; i < FS; ++i) accH[i] = accW[i] = 0.f;
#pragma unroll
  for (int k = 0; k < PP; ++k) {
    float cc = 0.f, g1 = 0.f;
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      const float bv = sB[c[k] + (i - P)];
      cc += fw[i] * bv;
      g1 += fh[i] * sG2[c[k] + (P - i) * Wp];
      // tap gradients: dFH[i] += G2[p] A[p shifted down by i-P], dFW[i] += G3[p] B[p shifted right]
      accH[i] += g2[k] * av[k][i];
      accW[i] += g[k] * bv;
    }
    if (ok[k]) {
      Cc[base + lane + 64 * k] = cc;
      G1[base + lane + 64 * k] = g1;
    }
  }
#pragma unroll
  for (int i = 0; i < FS; ++i) {
    accH[i] = wave_sum_to_lane63(accH[i]);
    accW[i] = wave_sum_to_lane63(accW[i]);
  }
  if (lane == 63) {
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      partH[((size_t)n * FS + i) * R + r] = accH[i];
      partW[((size_t)n * FS + i) * R + r] = accW[i];
    }
  }
}

// Border and size of the padded LDS planes of taps_wave_kernel.
struct WaveTapLayout {
  int Q, cells;
  size_t smem;
};
WaveTapLayout wave_tap_layout(int H, int W, int FS, int P) {
  WaveTapLayout l;
  l.Q = P > FS - 1 - P ? P : FS - 1 - P;
  const int raw = (H + 2 * l.Q) * (W + 2 * l.Q);
  l.cells = (raw + 3) & ~3;
  l.smem = (size_t)4 * 4 * l.cells * sizeof(float);
  return l;
}

template <int FS>
hipError_t launch_taps_wave(const float* A, const float* G3, const BwdFilterArgs& a, float* Cc,
                            float* G1, float* pH, float* pW, hipStream_t st) {
  const int HW = a.H * a.W, nplanes = a.N * a.R;
  const WaveTapLayout l = wave_tap_layout(a.H, a.W, FS, a.pad);
  const unsigned grid = (unsigned)((nplanes + 3) / 4);
  const unsigned wmagic = (unsigned)(0x100000000ull / (unsigned)a.W) + 1u;   // p / W for p < 65536
  const int PP = (HW + 63) / 64;
#define CP4_TW(pp)                                                                             \
  taps_wave_kernel<FS, pp><<<grid, 256, l.smem, st>>>(A, G3, a.FH, a.FW, Cc, G1, pH, pW, a.R, \
                                                      a.H, a.W, a.pad, l.Q, wmagic, nplanes)
  switch (PP) {
    case 1: CP4_TW(1); break;
    case 2: CP4_TW(2); break;
    case 3: CP4_TW(3); break;
    default: CP4_TW(4); break;
  }
#undef CP4_TW
  return hipGetLastError();
}

// ---- 2''. taps with lane = column: one wave per (image, rank) plane up to 64
// pixels wide; wider planes are cut into column segments of 64 - 2Q output
// columns (Q = max(P, FS-1-P), the reach of the horizontal taps), one wave per
// segment, whose 64 lanes also carry the Q halo columns on either side - read
// from memory like the others, so the shuffles below stay inside the wave - and
// which stores and sums only its own columns.  The wave walks down the rows.  The last FS rows of A, G3 and
// G2 live in registers; the horizontal taps read the neighbouring columns'
// registers through wave shuffles; nothing goes through LDS and there is no
// barrier.  Row t of A and G3 is requested kRowsAhead steps before it is used.
// Step t completes B and Cc on row t-(FS-1-P), G2 on row t, G1 on row t-P and
// the tap-gradient terms of row t-(FS-1-P).  Needs P <= FS-1.
constexpr int kRowsAhead = 8;
template <int FS>
__global__ __launch_bounds__(256) void taps_column_kernel(
    const float* __restrict__ A, const float* __restrict__ G3, const float* __restrict__ FH,
    const float* __restrict__ FW, float* __restrict__ Cc, float* __restrict__ G1,
    float* __restrict__ partH, float* __restrict__ partW, int R, int H, int W, int P,
    int nplanes, int segs, int Q, int rsegs, int RH) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int unit = blockIdx.x * 4 + wave;        // (plane, column segment, row segment)
  if (unit >= nplanes * segs * rsegs) return;
  const int pseg = unit / rsegs, rseg = unit - pseg * rsegs;
  const int plane = pseg / segs, seg = pseg - plane * segs;
  // Rows r0 .. r1-1 are this wave's: it stores and sums those only.  Its walk starts Q
  // rows above (the windows of its first outputs hold rows from r0 - Q on; what the
  // windows hold from further up is not used by any row it stores) and ends as the
  // whole-plane walk does.
  const int r0 = rseg * RH, r1 = min(H, r0 + RH);
  const int tstart = max(0, r0 - Q);
  const int r = plane % R, n = plane / R;
  const size_t base = (size_t)plane * H * W;
  // lane's image column; one segment: lane = column, no halo
  const int gc = segs == 1 ? lane : seg * (64 - 2 * Q) - Q + lane;
  const bool col = gc >= 0 && gc < W;
  // columns this wave stores and sums (the halo lanes belong to the neighbours)
  const bool mine = col && (segs == 1 || (lane >= Q && lane < 64 - Q));
  const int wc = gc < 0 ? 0 : (gc < W ? gc : W - 1);   // clamped column for addresses
  float fh[FS], fw[FS];
#pragma unroll
  for (int i = 0; i < FS; ++i) {
    fh[i] = FH[i * R + r];
    fw[i] = FW[i * R + r];
  }
  // source lanes of the horizontal taps; a tap that falls outside the row reads
  // lane 0 and is masked
  int srcf[FS], srcb[FS];
  bool okf[FS], okb[FS];
#pragma unroll
  for (int j = 0; j < FS; ++j) {
    const int wf = lane + j - P, wb = lane - j + P;   // forward / adjoint neighbour lane
    okf[j] = col && wf >= 0 && wf < 64 && gc + j - P >= 0 && gc + j - P < W;
    okb[j] = col && wb >= 0 && wb < 64 && gc - j + P >= 0 && gc - j + P < W;
    srcf[j] = okf[j] ? wf : 0;
    srcb[j] = okb[j] ? wb : 0;
  }
  float aw[FS], gw[FS], g2w[FS];                   // rows t-FS+1 .. t of A, G3, G2
#pragma unroll
  for (int i = 0; i < FS; ++i) aw[i] = gw[i] = g2w[i] = 0.f;
  float accH[FS], accW[FS];
#pragma unroll
  for (int i = 0; i < FS; ++i) accH[i] = accW[i] = 0.f;
  float ar[kRowsAhead], gr[kRowsAhead];
  auto request = [&](int slot, int row) {          // rows past the plane count as zero
    const int rc = row < H ? row : H - 1;
    ar[slot] = A[base + (size_t)rc * W + wc];
    gr[slot] = G3[base + (size_t)rc * W + wc];
  };
#pragma unroll
  for (int u = 0; u < kRowsAhead; ++u) request(u, tstart + u);
  const int tail = (FS - 1 - P) > P ? (FS - 1 - P) : P;
  for (int t0 = tstart; t0 < r1 + tail; t0 += kRowsAhead) {
#pragma unroll
    for (int u = 0; u < kRowsAhead; ++u) {
      const int t = t0 + u;
      if (t < r1 + tail) {
        const bool live = col && t < H;
        const float a_t = live ? ar[u] : 0.f, g_t = live ? gr[u] : 0.f;
        request(u, t + kRowsAhead);
        // G2 row t: horizontal adjoint taps of G3 row t
        float g2_t = 0.f;
#pragma unroll
        for (int j = 0; j < FS; ++j) {
          const float v = __shfl(g_t, srcb[j], 64);
          g2_t += okb[j] ? fw[j] * v : 0.f;
        }
#pragma unroll
        for (int i = 0; i + 1 < FS; ++i) {
          aw[i] = aw[i + 1];
          gw[i] = gw[i + 1];
          g2w[i] = g2w[i + 1];
        }
        aw[FS - 1] = a_t;
        gw[FS - 1] = g_t;
        g2w[FS - 1] = g2_t;
        // B, Cc and the tap-gradient terms of row hb
        const int hb = t - (FS - 1 - P);
        if (hb >= r0 && hb < r1) {
          float b = 0.f;
#pragma unroll
          for (int i = 0; i < FS; ++i) b += fh[i] * aw[i];
          float cc = 0.f;
#pragma unroll
          for (int j = 0; j < FS; ++j) {
            const float v = __shfl(b, srcf[j], 64);
            const float bj = okf[j] ? v : 0.f;
            cc += fw[j] * bj;
            accW[j] += mine ? gw[P] * bj : 0.f;     // G3[hb][w] * B[hb][w+j-P]
          }
#pragma unroll
          for (int i = 0; i < FS; ++i)
            accH[i] += mine ? g2w[P] * aw[i] : 0.f;   // G2[hb][w] * A[hb+i-P][w]
          if (mine) Cc[base + (size_t)hb * W + gc] = cc;
        }
        // G1 row hg: vertical adjoint taps of the G2 window
        const int hg = t - P;
        if (hg >= r0 && hg < r1) {
          float g1 = 0.f;
#pragma unroll
          for (int i = 0; i < FS; ++i) g1 += fh[i] * g2w[FS - 1 - i];
          if (mine) G1[base + (size_t)hg * W + gc] = g1;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < FS; ++i) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      accH[i] += __shfl_down(accH[i], off, 64);
      accW[i] += __shfl_down(accW[i], off, 64);
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      partH[((((size_t)n * segs + seg) * rsegs + rseg) * FS + i) * R + r] = accH[i];
      partW[((((size_t)n * segs + seg) * rsegs + rseg) * FS + i) * R + r] = accW[i];
    }
  }
}

// Column segments of taps_column_kernel for a plane W wide.
int column_segments(int W, int FS, int P) {
  const int Q = P > FS - 1 - P ? P : FS - 1 - P;
  return W <= 64 ? 1 : (W + (64 - 2 * Q) - 1) / (64 - 2 * Q);
}
// Rows per row segment: a wave walks its rows one after the other, so tall planes are
// cut until there are about 4096 waves, but not below 8 rows a segment (each walk
// starts with Q rows of the segment above).
int column_row_height(int N, int R, int H, int W, int FS, int P) {
  const long units = (long)N * R * column_segments(W, FS, P);
  long rsegs = (4096 + units - 1) / units;
  if (rsegs > H / 8) rsegs = H / 8;
  if (rsegs < 1) rsegs = 1;
  return (int)((H + rsegs - 1) / rsegs);
}
int column_row_segments(int N, int R, int H, int W, int FS, int P) {
  const int RH = column_row_height(N, R, H, W, FS, P);
  return (H + RH - 1) / RH;
}

template <int FS>
hipError_t launch_taps_column(const float* A, const float* G3, const BwdFilterArgs& a, float* Cc,
                              float* G1, float* pH, float* pW, hipStream_t st) {
  const int nplanes = a.N * a.R, segs = column_segments(a.W, FS, a.pad);
  const int Q = a.pad > FS - 1 - a.pad ? a.pad : FS - 1 - a.pad;
  const int RH = column_row_height(a.N, a.R, a.H, a.W, FS, a.pad);
  const int rsegs = (a.H + RH - 1) / RH;
  const long units = (long)nplanes * segs * rsegs;
  taps_column_kernel<FS><<<(unsigned)((units + 3) / 4), 256, 0, st>>>(
      A, G3, a.FH, a.FW, Cc, G1, pH, pW, a.R, a.H, a.W, a.pad, nplanes, segs, Q, rsegs, RH);
  return hipGetLastError();
}

// ---- 3a. partial[s][d][r] = sum_{p in split s} act[n,d,p] Z[n,r,p] ----------
struct GradArgs {
  const act_t* act[2];   // dy, x
  const float* Z[2];     // Cc, G1
  float* part[2];        // [S][D][R]
  int D[2];
  int N, R, RP, HW, PS, cps;   // PS pixel splits per image, cps 32-pixel chunks per split
  long long* dbg;
};

[[maybe_unused]] constexpr int kLd = 34;   // LDS row stride of the 32-pixel operand tiles (conflict-free)

#ifndef CP4_BWF_IO16
template <int RB>
__global__ __launch_bounds__(kCT) void grad_gemm_kernel(GradArgs a) {
  __shared__ float Zs[32 * RB * kLd];
  __shared__ float As[kCT / 64][32 * kLd];
  const int which = blockIdx.z;
  const int D = a.D[which], R = a.R, HW = a.HW;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  const int d0 = blockIdx.y * 128 + wave * 32;
  if ((int)blockIdx.y * 128 >= D) return;
  const int s = blockIdx.x, n = s / a.PS, ps = s - n * a.PS;
  const int nch_total = (HW + 31) >> 5;
  const int ch0 = ps * a.cps, ch1 = min(nch_total, ch0 + a.cps);
  const float* actn = a.act[which] + (size_t)n * D * HW;
  const float* zn = a.Z[which] + (size_t)n * R * HW;
  // tile loads: a lane moves float2; 16 lanes cover one 32-pixel row
  const int trow = lane >> 4, tcol = 2 * (lane & 15);
  float2 av[8], zv[RB * 2];
  auto load_tiles = [&](int ch) {
    const int p = ch * 32 + tcol;
    const bool pin = p < HW;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int d = d0 + 4 * j + trow;
      av[j] = (pin && d < D) ? *reinterpret_cast<const float2*>(actn + (size_t)d * HW + p)
                             : make_float2(0.f, 0.f);
    }
#pragma unroll
    for (int j = 0; j < RB * 2; ++j) {
      const int r = 16 * j + 4 * wave + trow;     // 4 waves x 4 rows per j
      zv[j] = (pin && r < R) ? *reinterpret_cast<const float2*>(zn + (size_t)r * HW + p)
                             : make_float2(0.f, 0.f);
    }
  };
  auto store_tiles = [&]() {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      *reinterpret_cast<float2*>(&As[wave][(4 * j + trow) * kLd + tcol]) = av[j];
#pragma unroll
    for (int j = 0; j < RB * 2; ++j)
      *reinterpret_cast<float2*>(&Zs[(16 * j + 4 * wave + trow) * kLd + tcol]) = zv[j];
  };
  f32x16 acc[RB];
#pragma unroll
  for (int mb = 0; mb < RB; ++mb) acc[mb] = (f32x16)(0.f);
  if (ch0 < ch1) load_tiles(ch0);
  for (int ch = ch0; ch < ch1; ++ch) {
    __syncthreads();              // previous chunk's MFMAs are done with the tiles
    store_tiles();
    __syncthreads();
    if (ch + 1 < ch1) load_tiles(ch + 1);   // in flight during the MFMAs
    const float* ap = &As[wave][l32 * kLd + hi];
    const float* zp = &Zs[l32 * kLd + hi];
#pragma unroll
    for (int st = 0; st < 16; ++st) {
      const float av1 = ap[2 * st];
#pragma unroll
      for (int mb = 0; mb < RB; ++mb) acc[mb] = mfma32(av1, zp[mb * 32 * kLd + 2 * st], acc[mb]);
    }
  }
  float* out = a.part[which] + (size_t)s * D * R;
#pragma unroll
  for (int mb = 0; mb < RB; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int d = d0 + 8 * (v >> 2) + 4 * hi + (v & 3), r = 32 * mb + l32;
      if (d < D && r < R) out[(size_t)d * R + r] = acc[mb][v];
    }
}

#endif  // !CP4_BWF_IO16

// ---- 3a'. the same gradient GEMMs as exact split-bf16 products (H*W a
// multiple of 4 so that rows can be moved as float4).  Per 32-pixel chunk the
// workgroup splits the Z tile once, cooperatively, straight from global memory
// into MFMA B fragments in LDS ([rank block][16-pixel step][part][half][rank] x
// 16 B, double-buffered: one barrier per chunk); every wave stages its own 32
// activation rows through a wave-private LDS tile (row-contiguous global reads)
// and splits them as the A operand.
constexpr int kLdS = 36;   // LDS row stride (floats) of the activation tile: 16-byte aligned rows

template <int RB, bool VEC>
__global__ __launch_bounds__(kCT) void grad_split_kernel(GradArgs a) {
  using namespace split;
  __shared__ __attribute__((aligned(16))) float As[kCT / 64][32 * kLdS];
  __shared__ u32x4 Zf[2][RB * 2 * 3 * 2 * 32];
  const int which = blockIdx.z;
  const int D = a.D[which], R = a.R, HW = a.HW;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  const int d0 = blockIdx.y * 128 + wave * 32;
  if ((int)blockIdx.y * 128 >= D) return;
  const int s = blockIdx.x, n = s / a.PS, ps = s - n * a.PS;
  [[maybe_unused]] const int dwg = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
  BSTAMP(a.dbg, 1, dwg, 4, 0)
  const int nch_total = (HW + 31) >> 5;
  const int ch0 = ps * a.cps, ch1 = min(nch_total, ch0 + a.cps);
  const act_t* actn = a.act[which] + (size_t)n * D * HW;
  const float* zn = a.Z[which] + (size_t)n * R * HW;
  // activation tile: lane moves float4; 8 lanes cover one 32-pixel row, 8 rows per load
  const int arow = lane >> 3, acol = 4 * (lane & 7);
  // Z tile: thread t splits the 8 pixels (octet zo) of rank row zr
  const int zr = tid >> 2, zo = tid & 3;             // 64 rows x 4 octets = 256 threads
  const bool zmine = zr < 32 * RB;
  float4 av[4], zv[2];
#ifdef CP4_BWF_IO16
  // four 16-bit activations (one 8-byte load when VEC) widened to fp32
  auto load4_act = [&](const act_t* row, int p) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (VEC) {
      if (p < HW) {
        const uint2 b = *reinterpret_cast<const uint2*>(row + p);
#ifdef CP4_BWF_HALF
        v.x = act_to_f32((act_t)(b.x & 0xffffu));
        v.y = act_to_f32((act_t)(b.x >> 16));
        v.z = act_to_f32((act_t)(b.y & 0xffffu));
        v.w = act_to_f32((act_t)(b.y >> 16));
#else
        v.x = __uint_as_float(b.x << 16);
        v.y = __uint_as_float(b.x & 0xffff0000u);
        v.z = __uint_as_float(b.y << 16);
        v.w = __uint_as_float(b.y & 0xffff0000u);
#endif
      }
    } else {
      if (p < HW) v.x = act_to_f32(row[p]);
      if (p + 1 < HW) v.y = act_to_f32(row[p + 1]);
      if (p + 2 < HW) v.z = act_to_f32(row[p + 2]);
      if (p + 3 < HW) v.w = act_to_f32(row[p + 3]);
    }
    return v;
  };
#endif
  // VEC: H*W is a multiple of 4 and the operands are 16-byte aligned, rows move
  // as float4; otherwise element by element with per-pixel bounds.
  auto load4 = [&](const float* row, int p) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (VEC) {
      if (p < HW) v = *reinterpret_cast<const float4*>(row + p);
    } else {
      if (p < HW) v.x = row[p];
      if (p + 1 < HW) v.y = row[p + 1];
      if (p + 2 < HW) v.z = row[p + 2];
      if (p + 3 < HW) v.w = row[p + 3];
    }
    return v;
  };
  auto load_tiles = [&](int ch) {
    const int p = ch * 32 + acol;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = d0 + 8 * j + arow;
#ifdef CP4_BWF_IO16
      av[j] = d < D ? load4_act(actn + (size_t)d * HW, p) : make_float4(0.f, 0.f, 0.f, 0.f);
#else
      av[j] = d < D ? load4(actn + (size_t)d * HW, p) : make_float4(0.f, 0.f, 0.f, 0.f);
#endif
    }
    const int pz = ch * 32 + 8 * zo;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      zv[j] = (zmine && zr < R) ? load4(zn + (size_t)zr * HW, pz + 4 * j)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
  };
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<float4*>(&As[wave][(8 * j + arow) * kLdS + acol]) = av[j];
    if (zmine) {
      const float v[8] = {zv[0].x, zv[0].y, zv[0].z, zv[0].w, zv[1].x, zv[1].y, zv[1].z, zv[1].w};
      u32x4 h, m, l;
      split8(v, h, m, l);
      // fragment (rank block zr/32, step zo/2, part, half zo&1, rank zr%32)
      u32x4* dst = &Zf[buf][(((zr >> 5) * 2 + (zo >> 1)) * 3 * 2 + (zo & 1)) * 32 + (zr & 31)];
      dst[0] = h;
      dst[64] = m;          // part stride: 2 halves x 32 ranks
      dst[128] = l;
    }
  };
  f32x16 acc[RB];
#pragma unroll
  for (int mb = 0; mb < RB; ++mb) acc[mb] = (f32x16)(0.f);
  if (ch0 < ch1) load_tiles(ch0);
  for (int ch = ch0; ch < ch1; ++ch) {
    const int buf = (ch - ch0) & 1;
    store_tiles(buf);
    if (ch - ch0 < 3) { BSTAMP(a.dbg, 1, dwg, 4, 1 + (ch - ch0)) }
    __syncthreads();        // Z fragments of this chunk are complete; the other buffer is free
    if (ch + 1 < ch1) load_tiles(ch + 1);   // in flight during the MFMAs
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const float* ap = &As[wave][l32 * kLdS + 16 * st + 8 * hi];
      const float4 a0 = *reinterpret_cast<const float4*>(ap);
      const float4 a1 = *reinterpret_cast<const float4*>(ap + 4);
      const float v[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#ifdef CP4_BWF_HALF
      // the activations are half-precision values: two bf16 parts
      u32x4 ah, am;
      split8_half(v, ah, am);
#pragma unroll
      for (int mb = 0; mb < RB; ++mb) {
        const u32x4* zp = &Zf[buf][((mb * 2 + st) * 3 * 2 + hi) * 32 + l32];
        acc[mb] = mfma16(ah, zp[128], acc[mb]);
        acc[mb] = mfma16(am, zp[64], acc[mb]);
        acc[mb] = mfma16(ah, zp[64], acc[mb]);
        acc[mb] = mfma16(am, zp[0], acc[mb]);
        acc[mb] = mfma16(ah, zp[0], acc[mb]);
      }
#elif defined(CP4_BWF_IO16)
      // the activations are bfloat16 values: their high part is all of them
      u32x4 ah;
#pragma unroll
      for (int d = 0; d < 4; ++d) ah[d] = pack_hi16(v[2 * d], v[2 * d + 1]);
#pragma unroll
      for (int mb = 0; mb < RB; ++mb) {
        const u32x4* zp = &Zf[buf][((mb * 2 + st) * 3 * 2 + hi) * 32 + l32];
        acc[mb] = mfma16(ah, zp[128], acc[mb]);
        acc[mb] = mfma16(ah, zp[64], acc[mb]);
        acc[mb] = mfma16(ah, zp[0], acc[mb]);
      }
#else
      u32x4 ah, am, al;
      split8(v, ah, am, al);
#pragma unroll
      for (int mb = 0; mb < RB; ++mb) {
        const u32x4* zp = &Zf[buf][((mb * 2 + st) * 3 * 2 + hi) * 32 + l32];
        acc[mb] = mfma_split(ah, am, al, zp[0], zp[64], zp[128], acc[mb]);
      }
#endif
    }
  }
  BSTAMP(a.dbg, 1, dwg, 4, 4)
  float* out = a.part[which] + (size_t)s * D * R;
#pragma unroll
  for (int mb = 0; mb < RB; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int d = d0 + 8 * (v >> 2) + 4 * hi + (v & 3), r = 32 * mb + l32;
      if (d < D && r < R) out[(size_t)d * R + r] = acc[mb][v];
    }
  BSTAMP(a.dbg, 1, dwg, 4, 5)
}

// ---- 3b. tap gradients: partial[s][t][r] over images of split s -------------

__global__ __launch_bounds__(256) void tap_grad_kernel(const float* __restrict__ G2,
                                                       const float* __restrict__ A,
                                                       const float* __restrict__ G3,
                                                       const float* __restrict__ B,
                                                       float* __restrict__ partH,
                                                       float* __restrict__ partW, int N, int R,
                                                       int H, int W, int Y, int X, int P, int S) {
  __shared__ float red[4];
  const int t = blockIdx.x, r = blockIdx.y, s = blockIdx.z;   // t < Y: dFH tap, else dFW tap
  const bool vertical = t < Y;
  const int tap = vertical ? t : t - Y, o = tap - P, HW = H * W;
  const float* P0 = vertical ? G2 : G3;
  const float* P1 = vertical ? A : B;
  const int n0 = (int)((long)N * s / S), n1 = (int)((long)N * (s + 1) / S);
  float acc = 0.f;
  for (int n = n0; n < n1; ++n) {
    const float* a = P0 + ((size_t)n * R + r) * HW;
    const float* b = P1 + ((size_t)n * R + r) * HW;
    for (int p = threadIdx.x; p < HW; p += 256) {
      const int h = p / W, w = p - h * W;
      const int hh = vertical ? h + o : h, ww = vertical ? w : w + o;
      if (hh >= 0 && hh < H && ww >= 0 && ww < W) acc += a[p] * b[hh * W + ww];
    }
  }
  const float tot = block_sum256(acc, red);
  if (threadIdx.x == 0) {
    if (vertical) partH[((size_t)s * Y + tap) * R + r] = tot;
    else partW[((size_t)s * X + tap) * R + r] = tot;
  }
}

// ---- 4. out[i] = sum_s partial[s][i], four segments in one launch -----------
struct ReduceArgs {
  const float* part[4];
  float* out[4];
  int count[4], S[4];
};
// A workgroup owns 64 consecutive outputs; its four waves each sum a quarter of
// the S partials in index order (eight loads in flight), then the four quarter
// sums are added in wave order: the result does not depend on timing.
__global__ __launch_bounds__(256) void reduce4_kernel(ReduceArgs a) {
  __shared__ float quarter[4][64];
  const int seg = blockIdx.y;
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + lane;
  const int count = a.count[seg], S = a.S[seg];
  if ((int)blockIdx.x * 64 >= count) return;               // whole workgroup
  const int k0 = (int)((long)S * q / 4), k1 = (int)((long)S * (q + 1) / 4);
  float s = 0.f;
  if (i < count) {
    const float* p = a.part[seg] + i;
    const size_t stride = count;
    int k = k0;
    for (; k + 8 <= k1; k += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = p[(size_t)(k + u) * stride];
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; k < k1; ++k) s += p[(size_t)k * stride];
  }
  quarter[q][lane] = s;
  __syncthreads();
  if (q == 0 && i < count)
    a.out[seg][i] = ((quarter[0][lane] + quarter[1][lane]) + quarter[2][lane]) + quarter[3][lane];
}

struct Plan {
  int RP, npb, PS, cps, S, St;
  bool plane_taps, wave_taps, column_taps;
  size_t plane, part_elems;
};
Plan make_plan(int N, int C, int T, int H, int W, int Y, int X, int R, int pad) {
  Plan p;
  const int HW = H * W;
  p.RP = R <= 32 ? 32 : 64;
  p.npb = (HW + 63) / 64;
  const int nch = (HW + 31) / 32;
  const int dgroups = (T + 127) / 128 + (C + 127) / 128;
  // Pixel splits per image: aim at 1024 workgroups (4 waves per SIMD hide the
  // load -> LDS -> MFMA latency of a chunk), but keep at least 6 chunks per split
  // so that the partials to write and sum stay small next to the operands.
  int PS = (1024 + N * dgroups - 1) / (N * dgroups);
  if (PS > nch / 6) PS = nch / 6;
  if (PS < 1) PS = 1;
  p.cps = (nch + PS - 1) / PS;
  p.PS = (nch + p.cps - 1) / p.cps;
  p.S = N * p.PS;
  p.plane_taps = (size_t)HW * 4 * sizeof(float) <= 64 * 1024 && Y + X <= 256;   // plane fits in LDS
  const bool odd_square = Y == X && (Y == 1 || Y == 3 || Y == 5 || Y == 7);
  p.wave_taps = p.plane_taps && HW <= 256 && W >= 2 && odd_square &&  // one wave per plane, in LDS
                wave_tap_layout(H, W, Y, pad).smem <= 64 * 1024;
  // one wave per plane (or per column segment of a wide plane), in registers
  p.column_taps = !p.wave_taps && odd_square && pad <= Y - 1;
  p.St = p.column_taps ? N * column_segments(W, Y, pad) * column_row_segments(N, R, H, W, Y, pad)
                       : (p.plane_taps ? N : (N < 8 ? N : 8));
  p.plane = (size_t)N * R * HW;
  // (tap partials: Y + X per plane, Y * X with the 3-factor op's depthwise filter)
  const size_t taps = (size_t)Y * X > (size_t)Y + X ? (size_t)Y * X : (size_t)Y + X;
  const size_t st_max = p.St > N ? p.St : N;
  p.part_elems = (size_t)p.S * R * ((size_t)T + C) + st_max * R * taps;
  return p;
}

}  // namespace

bool bwd_filter_mfma_supported(const cp4_shape& s) {
  // odd planes need the split contraction (scalar loads): channel counts multiples of 16
#ifdef CP4_BWF_IO16
  // the 16-bit builds have the split kernels only, one fragment tile of channels
  const bool odd_plane_ok = (s.C & 15) == 0 && (s.T & 15) == 0 &&
                            (size_t)(s.C > s.T ? s.C : s.T) * 192 <= 160 * 1024;
  if (!odd_plane_ok) return false;
#else
  const bool odd_plane_ok = (s.C & 15) == 0 && (s.T & 15) == 0;   // (more channels: in slices)
#endif
  return s.Rank <= 64 && fits_int_indexing((int)s.N, (int)s.H, (int)s.W) &&
         (((s.H * s.W) & 1) == 0 || odd_plane_ok) && (s.C & 1) == 0 &&
         (s.T & 1) == 0 && s.Y + s.X <= 65535;   // (any channel count: the factor tile is sliced)
}

#ifndef CP4_BWF_IO16
// The depthwise-filter tap step keeps two planes and Y*X partial sums in LDS.
bool bwd_filter_mfma_taps2d_supported(const cp4_shape& s) {
  return bwd_filter_mfma_supported(s) &&
         ((size_t)s.H * s.W * 2 + 5 * (size_t)s.Y * s.X) * sizeof(float) <= 64 * 1024;
}
#endif

size_t bwd_filter_mfma_workspace_bytes(const cp4_shape& s) {
  const Plan p = make_plan(s.N, s.C, s.T, s.H, s.W, s.Y, s.X, s.Rank, s.pad);
  return (6 * p.plane + p.part_elems) * sizeof(float);
}

hipError_t bwd_filter_mfma_launch(const BwdFilterArgs& a, hipStream_t st) {
  const int HW = a.H * a.W, R = a.R, N = a.N;
  const Plan p = make_plan(N, a.C, a.T, a.H, a.W, a.Y, a.X, R, a.pad);
  float* ws = static_cast<float*>(a.workspace);
  float *A = ws, *B = ws + p.plane, *Cc = ws + 2 * p.plane, *G3 = ws + 3 * p.plane,
        *G2 = ws + 4 * p.plane, *G1 = ws + 5 * p.plane, *part = ws + 6 * p.plane;
  float* pK = part;
  float* pC = pK + (size_t)p.S * a.T * R;
  float* pH = pC + (size_t)p.S * a.C * R;
  float* pW = pH + (size_t)p.St * a.Y * R;

  ContractArgs c{};
  // (bfloat16 build: BwdFilterArgs::x / dy point at 16-bit elements)
  const act_t* ax = reinterpret_cast<const act_t*>(a.x);
  const act_t* ady = reinterpret_cast<const act_t*>(a.dy);
  c.src[0] = ax; c.F[0] = a.FC; c.Z[0] = A; c.Cin[0] = a.C;
  c.src[1] = ady; c.F[1] = a.FK; c.Z[1] = G3; c.Cin[1] = a.T;
  c.N = N; c.R = R; c.RP = p.RP; c.HW = HW; c.npb = p.npb;
  c.items = N * p.npb;
#ifdef CP4_DEBUG_PHASES
  c.dbg = debug_stamp_buffer();
#endif
  const int cmax = a.C > a.T ? a.C : a.T;
  hipError_t e;
  if ((a.C & 15) == 0 && (a.T & 15) == 0 && (size_t)cmax * 192 <= 160 * 1024) {
    // exact split products: 32-pixel blocks, fragments of 6 bytes per factor entry
    c.npb = (HW + 31) / 32;
    c.items = N * c.npb;
    // few items: 2 or 4 waves per item, each on a slice of the channels, until
    // there are about 1024 waves (every workgroup builds the whole factor tile,
    // so more splits than that cost more than they hide; a slice keeps >= 2 chunks)
    c.ks = 1;
    const int nch_min = (a.C < a.T ? a.C : a.T) >> 4;
    while (c.ks < 4 && (long)c.items * 2 * (p.RP / 32) * c.ks < kKsWaves &&
           ((a.C >> 4) % (2 * c.ks)) == 0 && ((a.T >> 4) % (2 * c.ks)) == 0 &&
           nch_min / (2 * c.ks) >= 2)
      c.ks *= 2;
    size_t smem = (size_t)cmax * 192;
    if (c.ks > 1 && smem < (size_t)kSW * 16 * sizeof(float)) smem = (size_t)kSW * 16 * sizeof(float);
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(contract_split_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    const long slots = (long)c.items * c.ks;
    contract_split_kernel<<<dim3((unsigned)((slots + kSW / 64 - 1) / (kSW / 64)), 2, p.RP / 32),
                            kSW, smem, st>>>(c);
#ifndef CP4_BWF_IO16
  } else if ((a.C & 15) == 0 && (a.T & 15) == 0 && (HW & 1)) {
    // an odd plane (no float2 rows for the fp32 kernel below) with more channels than
    // the split kernel's fragment tile holds (853): the sum over channels runs a slice
    // of up to 768 at a time, each slice's contraction into the idle B plane and added
    // to its plane in slice order (the planes have R rows against hundreds of channels,
    // so the extra pass over them is cheap; N8 C2048 K512 7x7: 90 us, general kernel
    // 1085).  Even planes: one launch of the fp32 kernel, which slices its own factor
    // tile, is the quicker (N4 C1024 K2048 14x14 R48: 108 against 121 us).
    c.npb = (HW + 31) / 32;
    c.items = N * c.npb;
    c.ks = 1;
    for (int which = 0; which < 2; ++which) {
      const int Cin = which ? a.T : a.C;
      const int nsl = (Cin + kSplitSlice - 1) / kSplitSlice;
      const int cs = ((Cin + nsl - 1) / nsl + 15) / 16 * 16;
      float* Z = which ? G3 : A;
      for (int c0 = 0; c0 < Cin; c0 += cs) {
        ContractArgs d = c;
        d.src[0] = (which ? ady : ax) + (size_t)c0 * HW;
        d.F[0] = (which ? a.FK : a.FC) + (size_t)c0 * R;
        d.Z[0] = c0 ? B : Z;
        d.Cin[0] = Cin - c0 < cs ? Cin - c0 : cs;
        d.ldc[0] = Cin;
        const size_t smem = (size_t)d.Cin[0] * 192;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(contract_split_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return e;
        contract_split_kernel<<<dim3((unsigned)((c.items + kSW / 64 - 1) / (kSW / 64)), 1,
                                     p.RP / 32),
                                kSW, smem, st>>>(d);
        if (c0) {
          e = add_f32_launch(Z, B, (size_t)N * R * HW, st);
          if (e != hipSuccess) return e;
        }
      }
    }
#endif
  } else {
#ifdef CP4_BWF_IO16
    return hipErrorInvalidValue;      // excluded by bwd_filter_mfma_io16_supported
#else
    const size_t smem = (size_t)(cmax < kContractSlice ? cmax : kContractSlice) * 32 * sizeof(float);
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(contract_mfma_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    contract_mfma_kernel<<<dim3((c.items + kCW / 64 - 1) / (kCW / 64), 2, p.RP / 32), kCW, smem,
                           st>>>(c);
#endif
  }

  const bool wave_taps = p.wave_taps, column_taps = p.column_taps;
  if (a.taps2d) {
    const size_t tsm = ((size_t)HW * 2 + 5 * (size_t)a.Y * a.X) * sizeof(float);
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(taps2d_plane_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)tsm);
    if (e != hipSuccess) return e;
    taps2d_plane_kernel<<<N * R, 256, tsm, st>>>(A, G3, a.taps2d, Cc, G1, pH, R, a.H, a.W, a.Y,
                                                 a.X, a.pad);
  } else if (column_taps) {
    switch (a.Y) {
      case 1: e = launch_taps_column<1>(A, G3, a, Cc, G1, pH, pW, st); break;
      case 3: e = launch_taps_column<3>(A, G3, a, Cc, G1, pH, pW, st); break;
      case 5: e = launch_taps_column<5>(A, G3, a, Cc, G1, pH, pW, st); break;
      default: e = launch_taps_column<7>(A, G3, a, Cc, G1, pH, pW, st); break;
    }
    if (e != hipSuccess) return e;
  } else if (wave_taps) {
    switch (a.Y) {
      case 1: e = launch_taps_wave<1>(A, G3, a, Cc, G1, pH, pW, st); break;
      case 3: e = launch_taps_wave<3>(A, G3, a, Cc, G1, pH, pW, st); break;
      case 5: e = launch_taps_wave<5>(A, G3, a, Cc, G1, pH, pW, st); break;
      default: e = launch_taps_wave<7>(A, G3, a, Cc, G1, pH, pW, st); break;
    }
    if (e != hipSuccess) return e;
  } else if (p.plane_taps) {
    const size_t tsm = ((size_t)HW * 4 + 5 * (a.Y + a.X)) * sizeof(float);
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(taps_plane_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)tsm);
    if (e != hipSuccess) return e;
    taps_plane_kernel<<<N * R, 256, tsm, st>>>(A, G3, a.FH, a.FW, B, Cc, G2, G1, pH, pW, R, a.H,
                                               a.W, a.Y, a.X, a.pad);
  } else {
    taps_kernel<<<(unsigned)((p.plane + 255) / 256), 256, 0, st>>>(
        A, G3, a.FH, a.FW, B, Cc, G2, G1, p.plane, R, a.H, a.W, a.Y, a.X, a.pad);
    tap_grad_kernel<<<dim3(a.Y + a.X, R, p.St), 256, 0, st>>>(G2, A, G3, B, pH, pW, N, R, a.H,
                                                              a.W, a.Y, a.X, a.pad, p.St);
  }

  GradArgs g{};
  g.act[0] = ady; g.Z[0] = Cc; g.part[0] = pK; g.D[0] = a.T;
  g.act[1] = ax; g.Z[1] = G1; g.part[1] = pC; g.D[1] = a.C;
  g.N = N; g.R = R; g.RP = p.RP; g.HW = HW; g.PS = p.PS; g.cps = p.cps;
#ifdef CP4_DEBUG_PHASES
  g.dbg = debug_stamp_buffer();
#endif
  const int dmax = a.T > a.C ? a.T : a.C;
  const dim3 ggrid(p.S, (dmax + 127) / 128, 2);
  // rows of four pixels as one load: 16 bytes of fp32, 8 bytes of bfloat16
  const bool grad_split =
      (HW & 3) == 0 && (reinterpret_cast<uintptr_t>(ws) & 15) == 0 &&
      ((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.dy)) &
       (4 * sizeof(act_t) - 1)) == 0;
  if (grad_split) {
    if (p.RP == 32) grad_split_kernel<1, true><<<ggrid, kCT, 0, st>>>(g);
    else grad_split_kernel<2, true><<<ggrid, kCT, 0, st>>>(g);
#ifdef CP4_BWF_IO16
  } else {
    // the element-wise staging takes any plane size and alignment
    if (p.RP == 32) grad_split_kernel<1, false><<<ggrid, kCT, 0, st>>>(g);
    else grad_split_kernel<2, false><<<ggrid, kCT, 0, st>>>(g);
  }
#else
  } else if (HW & 1) {
    // odd planes: the float2 staging of the fp32 kernel does not apply
    if (p.RP == 32) grad_split_kernel<1, false><<<ggrid, kCT, 0, st>>>(g);
    else grad_split_kernel<2, false><<<ggrid, kCT, 0, st>>>(g);
  } else {
    if (p.RP == 32) grad_gemm_kernel<1><<<ggrid, kCT, 0, st>>>(g);
    else grad_gemm_kernel<2><<<ggrid, kCT, 0, st>>>(g);
  }
#endif

  ReduceArgs r{};
  const float* parts[4] = {pK, pC, pH, pW};
  float* outs[4] = {a.dFK, a.dFC, a.taps2d ? a.dtaps2d : a.dFH, a.dFW};
  const int counts[4] = {a.T * R, a.C * R, a.taps2d ? a.Y * a.X * R : a.Y * R,
                         a.taps2d ? 0 : a.X * R};
  const int Ss[4] = {p.S, p.S, a.taps2d ? N : p.St, p.St};
  int maxc = 0;
  for (int i = 0; i < 4; ++i) {
    r.part[i] = parts[i]; r.out[i] = outs[i]; r.count[i] = counts[i]; r.S[i] = Ss[i];
    if (counts[i] > maxc) maxc = counts[i];
  }
  reduce4_kernel<<<dim3((maxc + 63) / 64, 4), 256, 0, st>>>(r);
  return hipGetLastError();
}

#ifndef CP4_BWF_IO16
// ---- The same pass for a layer with a stride (and any zeros before the image) ----
// y[ho, wo] reads x at (sh*ho + i - pt, sw*wo + j - pl), so the planes come in two
// sizes: A = FC^T x and G1 (the adjoint taps of G3) on the input's H x W grid,
// G3 = FK^T dy and Cc (the taps of A at the kept positions) on the output's
// Ho x Wo grid.  The contraction and gradient-GEMM kernels above run once per
// operand, each on its own plane size; only the tap step is new:
//   Cc[ho,wo]  = sum_{i,j} FH[i] FW[j] A[sh*ho + i - pt, sw*wo + j - pl]
//   G1[h,w]    = sum_{i,j} FH[i] FW[j] G3[(h + pt - i) / sh, (w + pl - j) / sw]   (exact divisions only)
//   dFH[i]    += sum_{ho,wo} G3[ho,wo] sum_j FW[j] A[sh*ho + i - pt, sw*wo + j - pl]
//   dFW[j]    += sum_{ho,wo} G3[ho,wo] sum_i FH[i] A[sh*ho + i - pt, sw*wo + j - pl]
// (the reference's layers take strides, test/layers.py:264-279; its kernels do not).
namespace {

// One workgroup per (image, rank): both planes in LDS, tap-gradient partials
// partH[n][i][r], partW[n][j][r] summed in a fixed order.
__global__ __launch_bounds__(256) void taps_strided_plane_kernel(
    const float* __restrict__ A, const float* __restrict__ G3, const float* __restrict__ FH,
    const float* __restrict__ FW, float* __restrict__ Cc, float* __restrict__ G1,
    float* __restrict__ partH, float* __restrict__ partW, int R, int H, int W, int Ho, int Wo,
    int Y, int X, int sh, int sw, int pt, int pl_) {
  extern __shared__ float pl[];
  const int HW = H * W, HWo = Ho * Wo;
  float *sA = pl, *sG = pl + HW;
  float* red = sG + HWo;                          // [Y + X][4] wave partials
  float* fh = red + 4 * (Y + X);                  // this rank's tap weights, read once
  float* fw = fh + Y;
  const int plane = blockIdx.x, r = plane % R, n = plane / R;
  const size_t basef = (size_t)plane * HW, bases = (size_t)plane * HWo;
  for (int p = threadIdx.x; p < HW; p += 256) sA[p] = A[basef + p];
  for (int q = threadIdx.x; q < HWo; q += 256) sG[q] = G3[bases + q];
  if ((int)threadIdx.x < Y) fh[threadIdx.x] = FH[threadIdx.x * R + r];
  else if ((int)threadIdx.x < Y + X) fw[threadIdx.x - Y] = FW[(threadIdx.x - Y) * R + r];
  __syncthreads();
  // Cc on the output grid
  for (int q = threadIdx.x; q < HWo; q += 256) {
    const int ho = q / Wo, wo = q - ho * Wo;
    float cc = 0.f;
    for (int i = 0; i < Y; ++i) {
      const int hh = sh * ho + i - pt;
      if (hh < 0 || hh >= H) continue;
      float row = 0.f;
      for (int j = 0; j < X; ++j) {
        const int ww = sw * wo + j - pl_;
        if (ww >= 0 && ww < W) row += fw[j] * sA[hh * W + ww];
      }
      cc += fh[i] * row;
    }
    Cc[bases + q] = cc;
  }
  // G1 on the input grid: the adjoint taps of G3
  for (int p = threadIdx.x; p < HW; p += 256) {
    const int h = p / W, w = p - h * W;
    float g1 = 0.f;
    for (int i = 0; i < Y; ++i) {
      const int num = h + pt - i;
      if (num < 0) break;
      const int ho = num / sh;
      if (ho * sh != num || ho >= Ho) continue;
      float row = 0.f;
      for (int j = 0; j < X; ++j) {
        const int numw = w + pl_ - j;
        if (numw < 0) break;
        const int wo = numw / sw;
        if (wo * sw == numw && wo < Wo) row += fw[j] * sG[ho * Wo + wo];
      }
      g1 += fh[i] * row;
    }
    G1[basef + p] = g1;
  }
  // tap gradients of this plane: wave sums to LDS, one barrier, then a fixed-order
  // sum of the four wave partials per tap
  for (int t = 0; t < Y + X; ++t) {
    const bool vertical = t < Y;
    float acc = 0.f;
    for (int q = threadIdx.x; q < HWo; q += 256) {
      const int ho = q / Wo, wo = q - ho * Wo;
      float inner = 0.f;
      if (vertical) {
        const int hh = sh * ho + t - pt;
        if (hh >= 0 && hh < H)
          for (int j = 0; j < X; ++j) {
            const int ww = sw * wo + j - pl_;
            if (ww >= 0 && ww < W) inner += fw[j] * sA[hh * W + ww];
          }
      } else {
        const int ww = sw * wo + (t - Y) - pl_;
        if (ww >= 0 && ww < W)
          for (int i = 0; i < Y; ++i) {
            const int hh = sh * ho + i - pt;
            if (hh >= 0 && hh < H) inner += fh[i] * sA[hh * W + ww];
          }
      }
      acc += sG[q] * inner;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if ((threadIdx.x & 63) == 0) red[t * 4 + (threadIdx.x >> 6)] = acc;
  }
  __syncthreads();
  if ((int)threadIdx.x < Y + X) {
    const int t = threadIdx.x;
    const float tot = red[t * 4] + red[t * 4 + 1] + red[t * 4 + 2] + red[t * 4 + 3];
    if (t < Y) partH[((size_t)n * Y + t) * R + r] = tot;
    else partW[((size_t)n * X + (t - Y)) * R + r] = tot;
  }
}

// The same for square filters of a compile-time size: the tap-gradient terms are
// accumulated in registers while Cc is formed (one pass over the plane instead of
// one per tap), and the adjoint taps are walked per block of sh x sw input pixels.
template <int FS>
__global__ __launch_bounds__(256) void taps_strided_fast_kernel(
    const float* __restrict__ A, const float* __restrict__ G3, const float* __restrict__ FH,
    const float* __restrict__ FW, float* __restrict__ Cc, float* __restrict__ G1,
    float* __restrict__ partH, float* __restrict__ partW, int R, int H, int W, int Ho, int Wo,
    int sh, int sw, int pt, int pl_) {
  constexpr int Y = FS, X = FS;
  extern __shared__ float pl[];
  const int HW = H * W, HWo = Ho * Wo;
  float *sA = pl, *sG = pl + HW;
  float* red = sG + HWo;                          // [Y + X][4] wave partials
  float* fh = red + 4 * (Y + X);                  // this rank's tap weights, read once
  float* fw = fh + Y;
  const int plane = blockIdx.x, r = plane % R, n = plane / R;
  const size_t basef = (size_t)plane * HW, bases = (size_t)plane * HWo;
  // planes into LDS, four pixels per load where the plane sizes allow (all of a
  // thread's loads are then in flight together)
  auto stage = [&](float* dst, const float* src, int n) {
    if ((n & 3) == 0 && ((reinterpret_cast<uintptr_t>(src) | (uintptr_t)(dst - pl) * 4) & 15) == 0) {
      const float4* s4 = reinterpret_cast<const float4*>(src);
      float4* d4 = reinterpret_cast<float4*>(dst);
#pragma unroll 4
      for (int k = threadIdx.x; k < (n >> 2); k += 256) d4[k] = s4[k];
    } else {
      for (int k = threadIdx.x; k < n; k += 256) dst[k] = src[k];
    }
  };
  stage(sA, A + basef, HW);
  stage(sG, G3 + bases, HWo);
  if ((int)threadIdx.x < Y) fh[threadIdx.x] = FH[threadIdx.x * R + r];
  else if ((int)threadIdx.x < Y + X) fw[threadIdx.x - Y] = FW[(threadIdx.x - Y) * R + r];
  __syncthreads();
  // Cc on the output grid, and this thread's share of the tap gradients.  Reads
  // outside the image go to a clamped cell and count zero: no branches, so the FS*FS
  // LDS reads of a pixel are all in flight together.
  float gh[FS], gw[FS];
#pragma unroll
  for (int t = 0; t < FS; ++t) gh[t] = gw[t] = 0.f;
  for (int q = threadIdx.x; q < HWo; q += 256) {
    const int ho = q / Wo, wo = q - ho * Wo;
    const float gv = sG[q];
    int ro[FS], co[FS];
    bool rin[FS], cin[FS];
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      const int hh = sh * ho + i - pt, ww = sw * wo + i - pl_;
      rin[i] = hh >= 0 && hh < H;
      cin[i] = ww >= 0 && ww < W;
      ro[i] = rin[i] ? hh * W : 0;
      co[i] = cin[i] ? ww : 0;
    }
    float av[FS][FS];
#pragma unroll
    for (int i = 0; i < FS; ++i)
#pragma unroll
      for (int j = 0; j < FS; ++j) av[i][j] = sA[ro[i] + co[j]];
    float cc = 0.f, col[FS];
#pragma unroll
    for (int j = 0; j < FS; ++j) col[j] = 0.f;
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      float row = 0.f;
#pragma unroll
      for (int j = 0; j < FS; ++j) {
        const float v = (rin[i] && cin[j]) ? av[i][j] : 0.f;
        row += fw[j] * v;
        col[j] += fh[i] * v;
      }
      cc += fh[i] * row;
      gh[i] += gv * row;
    }
#pragma unroll
    for (int j = 0; j < FS; ++j) gw[j] += gv * col[j];
    Cc[bases + q] = cc;
  }
  // G1 on the input grid: the adjoint taps of G3.  A thread takes a block of sh x sw
  // input pixels (bh, bw): tap row i lands on the block's row ai[i] = (i - pt) mod sh
  // and reads output row bh + dh[i] (both the same for every block), likewise for the
  // columns - so a block costs FS*FS reads in all, whichever of its pixels they go to.
  int ai[FS], dh[FS], bj[FS], dw[FS];
#pragma unroll
  for (int i = 0; i < FS; ++i) {
    ai[i] = ((i - pt) % sh + sh) % sh;
    dh[i] = (ai[i] + pt - i) / sh;               // exact
    bj[i] = ((i - pl_) % sw + sw) % sw;
    dw[i] = (bj[i] + pl_ - i) / sw;
  }
  const int nbw = (W + sw - 1) / sw, nbh = (H + sh - 1) / sh;
  for (int blk = threadIdx.x; blk < nbh * nbw; blk += 256) {
    const int bh = blk / nbw, bw = blk - bh * nbw;
    // the FS*FS values of G3 the block's pixels draw on (0 outside the plane), once
    float gv[FS][FS];
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      const int ho = bh + dh[i];
      const bool rok = ho >= 0 && ho < Ho;
#pragma unroll
      for (int j = 0; j < FS; ++j) {
        const int wo = bw + dw[j];
        const bool ok = rok && wo >= 0 && wo < Wo;
        const float v = sG[ok ? ho * Wo + wo : 0];
        gv[i][j] = ok ? v : 0.f;
      }
    }
    // pixel (a, b) of the block takes the taps that land on it: weights of the others 0
    for (int a = 0; a < sh; ++a) {
      const int h = sh * bh + a;
      if (h >= H) break;
      float wr[FS];
#pragma unroll
      for (int i = 0; i < FS; ++i) wr[i] = ai[i] == a ? fh[i] : 0.f;
      for (int b = 0; b < sw; ++b) {
        const int w = sw * bw + b;
        if (w >= W) break;
        float g1 = 0.f;
#pragma unroll
        for (int i = 0; i < FS; ++i) {
          float row = 0.f;
#pragma unroll
          for (int j = 0; j < FS; ++j) row += (bj[j] == b ? fw[j] : 0.f) * gv[i][j];
          g1 += wr[i] * row;
        }
        G1[basef + (size_t)h * W + w] = g1;
      }
    }
  }
  // wave sums of the tap gradients to LDS, one barrier, fixed-order sum of the four
#pragma unroll
  for (int t = 0; t < FS; ++t) {
    float a = gh[t], b = gw[t];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      a += __shfl_down(a, off, 64);
      b += __shfl_down(b, off, 64);
    }
    if ((threadIdx.x & 63) == 0) {
      red[t * 4 + (threadIdx.x >> 6)] = a;
      red[(Y + t) * 4 + (threadIdx.x >> 6)] = b;
    }
  }
  __syncthreads();
  if ((int)threadIdx.x < Y + X) {
    const int t = threadIdx.x;
    const float tot = red[t * 4] + red[t * 4 + 1] + red[t * 4 + 2] + red[t * 4 + 3];
    if (t < Y) partH[((size_t)n * Y + t) * R + r] = tot;
    else partW[((size_t)n * X + (t - Y)) * R + r] = tot;
  }
}

size_t strided_taps_lds(int H, int W, int Ho, int Wo, int Y, int X) {
  return ((size_t)H * W + (size_t)Ho * Wo + 5 * (size_t)(Y + X)) * sizeof(float);
}

// One channel -> rank contraction Z[n,r,p] = sum_c F[c,r] src[n,c,p] on planes of HW pixels.
hipError_t contract_one(const float* src, const float* F, float* Z, int Cin, int N, int R, int RP,
                        int HW, hipStream_t st) {
  ContractArgs c{};
  c.src[0] = src; c.F[0] = F; c.Z[0] = Z; c.Cin[0] = Cin;
  c.N = N; c.R = R; c.RP = RP; c.HW = HW;
  hipError_t e;
  if ((Cin & 15) == 0 && (size_t)Cin * 192 <= 160 * 1024) {
    c.npb = (HW + 31) / 32;
    c.items = N * c.npb;
    c.ks = 1;
    while (c.ks < 4 && (long)c.items * (RP / 32) * c.ks < kKsWaves / 2 &&
           ((Cin >> 4) % (2 * c.ks)) == 0 && (Cin >> 4) / (2 * c.ks) >= 2)
      c.ks *= 2;
    size_t smem = (size_t)Cin * 192;
    if (c.ks > 1 && smem < (size_t)kSW * 16 * sizeof(float)) smem = (size_t)kSW * 16 * sizeof(float);
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(contract_split_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    const long slots = (long)c.items * c.ks;
    contract_split_kernel<<<dim3((unsigned)((slots + kSW / 64 - 1) / (kSW / 64)), 1, RP / 32), kSW,
                            smem, st>>>(c);
  } else {
    c.npb = (HW + 63) / 64;
    c.items = N * c.npb;
    const size_t smem = (size_t)(Cin < kContractSlice ? Cin : kContractSlice) * 32 * sizeof(float);
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(contract_mfma_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    contract_mfma_kernel<<<dim3((c.items + kCW / 64 - 1) / (kCW / 64), 1, RP / 32), kCW, smem,
                           st>>>(c);
  }
  return hipGetLastError();
}

// One gradient GEMM part[s][d][r] = sum_{p in split s} act[n,d,p] Z[n,r,p] on planes of HW pixels.
hipError_t grad_one(const float* act, const float* Z, float* part, int D, int N, int R,
                    const Plan& p, int HW, const void* ws, hipStream_t st) {
  GradArgs g{};
  g.act[0] = act; g.Z[0] = Z; g.part[0] = part; g.D[0] = D;
  g.N = N; g.R = R; g.RP = p.RP; g.HW = HW; g.PS = p.PS; g.cps = p.cps;
  const dim3 ggrid(p.S, (D + 127) / 128, 1);
  const bool vec = (HW & 3) == 0 && (reinterpret_cast<uintptr_t>(ws) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(act) & 15) == 0;
  if (vec) {
    if (p.RP == 32) grad_split_kernel<1, true><<<ggrid, kCT, 0, st>>>(g);
    else grad_split_kernel<2, true><<<ggrid, kCT, 0, st>>>(g);
  } else if (HW & 1) {
    if (p.RP == 32) grad_split_kernel<1, false><<<ggrid, kCT, 0, st>>>(g);
    else grad_split_kernel<2, false><<<ggrid, kCT, 0, st>>>(g);
  } else {
    if (p.RP == 32) grad_gemm_kernel<1><<<ggrid, kCT, 0, st>>>(g);
    else grad_gemm_kernel<2><<<ggrid, kCT, 0, st>>>(g);
  }
  return hipGetLastError();
}

struct StridedLayout {
  Plan pf, ps;                                    // plans on the input's and on the output's grid
  size_t A, G1, G3, Cc, pK, pC, pH, pW, total;    // float offsets into the workspace
};
StridedLayout strided_layout(const cp4_shape& s, const Geometry& g) {
  StridedLayout l;
  l.pf = make_plan(s.N, s.C, s.T, s.H, s.W, s.Y, s.X, s.Rank, 0);
  l.ps = make_plan(s.N, s.C, s.T, g.Ho, g.Wo, s.Y, s.X, s.Rank, 0);
  const size_t planef = (size_t)s.N * s.Rank * s.H * s.W, planes = (size_t)s.N * s.Rank * g.Ho * g.Wo;
  auto al = [](size_t v) { return (v + 63) & ~(size_t)63; };   // 256-byte steps
  size_t o = 0;
  l.A = o; o += al(planef);
  l.G1 = o; o += al(planef);
  l.G3 = o; o += al(planes);
  l.Cc = o; o += al(planes);
  l.pK = o; o += al((size_t)l.ps.S * s.T * s.Rank);
  l.pC = o; o += al((size_t)l.pf.S * s.C * s.Rank);
  l.pH = o; o += al((size_t)s.N * s.Y * s.Rank);
  l.pW = o; o += al((size_t)s.N * s.X * s.Rank);
  l.total = o;
  return l;
}

}  // namespace

bool bwd_filter_mfma_strided_supported(const cp4_shape& s, const Geometry& g) {
  cp4_shape so = s;
  so.H = g.Ho; so.W = g.Wo;
  return bwd_filter_mfma_supported(s) && bwd_filter_mfma_supported(so) && s.Y + s.X <= 256 &&
         strided_taps_lds(s.H, s.W, g.Ho, g.Wo, s.Y, s.X) <= 150 * 1024;
}

size_t bwd_filter_mfma_strided_workspace_bytes(const cp4_shape& s, const Geometry& g) {
  return strided_layout(s, g).total * sizeof(float);
}

hipError_t bwd_filter_mfma_strided_launch(const BwdFilterArgs& a, const Geometry& g,
                                          hipStream_t st) {
  cp4_shape s{};
  s.N = a.N; s.C = a.C; s.T = a.T; s.H = a.H; s.W = a.W; s.pad = 0; s.Y = a.Y; s.X = a.X;
  s.Rank = a.R;
  const StridedLayout l = strided_layout(s, g);
  float* ws = static_cast<float*>(a.workspace);
  float *A = ws + l.A, *G1 = ws + l.G1, *G3 = ws + l.G3, *Cc = ws + l.Cc, *pK = ws + l.pK,
        *pC = ws + l.pC, *pH = ws + l.pH, *pW = ws + l.pW;
  const int N = a.N, R = a.R, HW = a.H * a.W, HWo = g.Ho * g.Wo;
  hipError_t e = contract_one(a.x, a.FC, A, a.C, N, R, l.pf.RP, HW, st);
  if (e != hipSuccess) return e;
  e = contract_one(a.dy, a.FK, G3, a.T, N, R, l.ps.RP, HWo, st);
  if (e != hipSuccess) return e;
  const size_t tsm = strided_taps_lds(a.H, a.W, g.Ho, g.Wo, a.Y, a.X);
  const bool fast = a.Y == a.X && (a.Y == 1 || a.Y == 3 || a.Y == 5 || a.Y == 7);
#define CP4_STRIDED_TAPS(FS_)                                                                    \
  {                                                                                              \
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(taps_strided_fast_kernel<FS_>),        \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)tsm);               \
    if (e != hipSuccess) return e;                                                               \
    taps_strided_fast_kernel<FS_><<<N * R, 256, tsm, st>>>(A, G3, a.FH, a.FW, Cc, G1, pH, pW, R, \
                                                           a.H, a.W, g.Ho, g.Wo, g.sh, g.sw,     \
                                                           g.pt, g.pl);                          \
  }
  if (fast) {
    switch (a.Y) {
      case 1: CP4_STRIDED_TAPS(1) break;
      case 3: CP4_STRIDED_TAPS(3) break;
      case 5: CP4_STRIDED_TAPS(5) break;
      default: CP4_STRIDED_TAPS(7) break;
    }
  } else {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(taps_strided_plane_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)tsm);
    if (e != hipSuccess) return e;
    taps_strided_plane_kernel<<<N * R, 256, tsm, st>>>(A, G3, a.FH, a.FW, Cc, G1, pH, pW, R, a.H,
                                                       a.W, g.Ho, g.Wo, a.Y, a.X, g.sh, g.sw, g.pt,
                                                       g.pl);
  }
#undef CP4_STRIDED_TAPS
  e = grad_one(a.dy, Cc, pK, a.T, N, R, l.ps, HWo, ws, st);
  if (e != hipSuccess) return e;
  e = grad_one(a.x, G1, pC, a.C, N, R, l.pf, HW, ws, st);
  if (e != hipSuccess) return e;
  ReduceArgs r{};
  const float* parts[4] = {pK, pC, pH, pW};
  float* outs[4] = {a.dFK, a.dFC, a.dFH, a.dFW};
  const int counts[4] = {a.T * R, a.C * R, a.Y * R, a.X * R};
  const int Ss[4] = {l.ps.S, l.pf.S, N, N};
  int maxc = 0;
  for (int i = 0; i < 4; ++i) {
    r.part[i] = parts[i]; r.out[i] = outs[i]; r.count[i] = counts[i]; r.S[i] = Ss[i];
    if (counts[i] > maxc) maxc = counts[i];
  }
  reduce4_kernel<<<dim3((maxc + 63) / 64, 4), 256, 0, st>>>(r);
  return hipGetLastError();
}
#endif  // !CP4_BWF_IO16

}  // namespace cp4
