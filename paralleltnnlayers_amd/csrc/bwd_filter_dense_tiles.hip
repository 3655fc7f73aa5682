// Backward-filter for layers with few channels on both sides: the dense filter gradient
//   dK[k,c,i,j] = sum_{n,h,w} dy[n,k,h,w] * x[n,c,h+i-pad,w+j-pad]
// over tiles of pixels, then the chain rule onto the four factors
//   dFK[k,r] = sum_{c,i,j} dK[k,c,i,j] FC[c,r] FH[i,r] FW[j,r]   (and likewise dFC, dFH, dFW),
// which is what Cuda_kernels/cp4Conv2dBackwardFilter.cu:64-257 computes factor by factor.
//
// With few channels the factor-by-factor order is the expensive one: its intermediates are
// [N, R, H, W] planes, sixteen ranks of them where x has three channels, and four kernels move
// them through memory (N16 C3 K1 512x512 R16: 67 MB of activations, 1.0 ms).  The dense
// gradient has K*C*Y*X entries (27 there), needs x and dy once and no intermediate at all.
//
//   1. a tile kernel, one of two (use_mfma): dense_mfma_kernel, the sums as a GEMM over the
//      pixels on the matrix cores, described where it is defined, or
//      dense_tiles_kernel<FS, KB>: persistent workgroups of 256 threads over tiles of
//      TH x TW pixels; the x tile with its halo and the dy tile go to LDS (zero outside the
//      image); a thread owns KB output channels x 4 input channels x FS x FS taps in
//      registers and a run of consecutive pixels of one row, along which the FS x FS window of
//      x slides (FS new cells per channel and pixel); partial sums stay in registers across a
//      workgroup's tiles, are added over the threads that share a channel block through LDS in
//      fixed order, and leave as one partial set per workgroup.
//   2. dense_reduce_kernel: the partial sets summed in fixed order.
//   3. dense_fold_kernel: the chain rule, a workgroup per 32 ranks and gradient.
// No atomics: bit-reproducible.  Plain fp32 multiply-adds, or exact fp32 products from bf16
// parts on the matrix cores.
#include "cp4_internal.h"
#include <atomic>
#include "split_bf16.h"

namespace cp4 {
namespace {

using split::f32x16;
using split::u32x4;

constexpr int kThreads = 256;
constexpr int kCB = 4;                       // input channels per thread
constexpr int kMaxPairs = 256;               // T * C up to here
constexpr int kMaxGrid = 1024;               // partial sets (up to four workgroups per compute unit)
constexpr size_t kLdsLimit = 64 * 1024;

struct DensePlan {
  int TH, TW, tilesX, tilesY, ntiles;
  int KBLK, CBLK;      // blocks of KB output channels / 4 input channels
  int G, S;            // channel-block groups; threads (pixel runs) per group
  int L;               // pixels per run
  int XS, XR;          // x tile in LDS: row stride (odd), rows * XS per channel
  int XSg, DRS;        // columns staged per row of x; row stride of the dy tile (odd)
  int skew;            // runs to lanes: four runs of a row, then the next row (see the kernel)
  int vec, xlead;      // 16-byte loads; columns of x staged before the tile's first (pad, or 4)
  int Cp, Tp;          // channel counts padded to their blocks
  int outs;            // T * C * FS * FS
  int lgTW, lgtile;    // log2 of TW and of TH * TW
  unsigned chmagic;    // ceil(2^32 / ((TH + FS - 1) * XSg))
  unsigned xsmagic;    // ceil(2^32 / XSg)
  int gbatch;          // groups whose partial sums the LDS holds at a time in the final sum
  int grid;
  size_t lds_bytes;
};

// A workgroup's tiles.  Workgroups go to the chip's eight dies in turn (blockIdx & 7), each die
// with an L2 of its own: a die takes one contiguous eighth of the tiles and its workgroups
// stride through it, so that tiles which share halo rows and columns run on the same die at
// about the same time (tile t, t + 1 on neighbouring dies: every halo cell is fetched once
// per die that needs it, 1.7 - 1.9 times the input in all).
struct TileRange {
  int first, end, step;
};
__device__ __forceinline__ TileRange tiles_of_workgroup(int ntiles) {
  const int dies = gridDim.x < 8 ? (int)gridDim.x : 8;            // (fewer than eight workgroups: a range each)
  const int die = blockIdx.x % dies, slot = blockIdx.x / dies;
  const int on_die = ((int)gridDim.x - die + dies - 1) / dies;     // workgroups on this die
  TileRange r;
  r.first = (int)((long)ntiles * die / dies) + slot;
  r.end = (int)((long)ntiles * (die + 1) / dies);
  r.step = on_die;
  return r;
}

template <int FS, int KB>
__global__ __launch_bounds__(kThreads) void dense_tiles_kernel(BwdFilterArgs a, DensePlan pl,
                                                               float* partial) {
  extern __shared__ float lds[];
  float* X = lds;                                    // [Cp][TH + FS - 1][XS]
  float* D = lds + (size_t)pl.Cp * pl.XR;            // [Tp][TH][DRS]
  const int DK = pl.TH * pl.DRS;                     // an output channel's tile
  const int tid = threadIdx.x;
  const int H = a.H, W = a.W, HW = H * W;
  const int PH = pl.TH + FS - 1, PW = pl.TW + FS - 1;
  // this thread: channel-block group g (output-channel block kb, input-channel block cb) and
  // run s of the tile's pixels
  const int g = tid / pl.S, s = tid - g * pl.S;
  const bool active = g < pl.G;
  const int kb = active ? g / pl.CBLK : 0, cb = active ? g - kb * pl.CBLK : 0;
  const int runs_per_row = pl.TW / pl.L;
  float acc[KB][kCB][FS][FS];
#pragma unroll
  for (int k = 0; k < KB; ++k)
#pragma unroll
    for (int c = 0; c < kCB; ++c)
#pragma unroll
      for (int i = 0; i < FS; ++i)
#pragma unroll
        for (int j = 0; j < FS; ++j) acc[k][c][i][j] = 0.f;

  // the channels that pad x to a multiple of four are zeros for the whole launch
  for (int e = a.C * pl.XR + tid; e < pl.Cp * pl.XR; e += kThreads) X[e] = 0.f;
  const int tiles_per_image = pl.tilesX * pl.tilesY;
  const TileRange tr = tiles_of_workgroup(pl.ntiles);
  for (int t = tr.first; t < tr.end; t += tr.step) {
    const int n = t / tiles_per_image, rem = t - n * tiles_per_image;
    const int ty = rem / pl.tilesX, tx = rem - ty * pl.tilesX;
    const int h0 = ty * pl.TH, w0 = tx * pl.TW;
    // ---- stage the x tile with its halo and the dy tile (zeros outside the image) ----
    // Whole LDS rows of XS cells: the cells past the plane's PW columns, which a run's last
    // steps may read, are zeros too.  Divisions by multiplication and shifts; eight loads in
    // flight per thread and batch (issued one by one each would wait out a memory round trip
    // of its own): addresses clamped, values selected, so that no load sits in a branch.
    constexpr int kBatch = 8;
    const float* xn = a.x + (size_t)n * a.C * HW;
    const float* dn = a.dy + (size_t)n * a.T * HW;
    const int nx = a.C * PH * pl.XSg;
    const int nd = pl.Tp * pl.TH * pl.TW;
    if (pl.vec) {
      // Four cells a load (W a multiple of four, x and dy 16-byte aligned): the tile's rows
      // start four columns before its first, so that a group of four is inside the image
      // together or not at all; four loads in flight per thread and batch.
      constexpr int kBatch4 = 4;
      for (int e0 = 4 * tid; e0 < nx; e0 += 4 * kThreads * kBatch4) {
        float4 v[kBatch4];
        int at[kBatch4];
        bool in[kBatch4];
#pragma unroll
        for (int u = 0; u < kBatch4; ++u) {
          const int e = e0 + 4 * u * kThreads;
          const int c = (int)__umulhi((unsigned)e, pl.chmagic), r2 = e - c * (PH * pl.XSg);
          const int pr = (int)__umulhi((unsigned)r2, pl.xsmagic), pc = r2 - pr * pl.XSg;
          const int h = h0 - a.pad + pr, w = w0 - 4 + pc;
          in[u] = e < nx && c < a.C && h >= 0 && h < H && w >= 0 && w < W;
          at[u] = e < nx ? c * pl.XR + pr * pl.XS + pc : -1;
          const int cc = c < a.C ? c : a.C - 1;
          const int hc = h < 0 ? 0 : (h > H - 1 ? H - 1 : h), wc = w < 0 ? 0 : (w > W - 4 ? W - 4 : w);
          v[u] = *reinterpret_cast<const float4*>(xn + (size_t)cc * HW + (size_t)hc * W + wc);
        }
#pragma unroll
        for (int u = 0; u < kBatch4; ++u)
          if (at[u] >= 0) {              // (rows an odd number of cells apart: four 4-byte stores)
            const float4 w4 = in[u] ? v[u] : make_float4(0.f, 0.f, 0.f, 0.f);
            X[at[u]] = w4.x; X[at[u] + 1] = w4.y; X[at[u] + 2] = w4.z; X[at[u] + 3] = w4.w;
          }
      }
      for (int e0 = 4 * tid; e0 < nd; e0 += 4 * kThreads * kBatch4) {
        float4 v[kBatch4];
        bool in[kBatch4];
        int at[kBatch4];
#pragma unroll
        for (int u = 0; u < kBatch4; ++u) {
          const int e = e0 + 4 * u * kThreads;
          const int k = e >> pl.lgtile, r2 = e & ((1 << pl.lgtile) - 1);
          const int pr = r2 >> pl.lgTW, pc = r2 & (pl.TW - 1);
          const int h = h0 + pr, w = w0 + pc;
          at[u] = e < nd ? k * DK + pr * pl.DRS + pc : -1;
          in[u] = e < nd && k < a.T && h < H && w < W;
          const int kc = k < a.T ? k : a.T - 1, hc = h > H - 1 ? H - 1 : h, wc = w > W - 4 ? W - 4 : w;
          v[u] = *reinterpret_cast<const float4*>(dn + (size_t)kc * HW + (size_t)hc * W + wc);
        }
#pragma unroll
        for (int u = 0; u < kBatch4; ++u)
          if (at[u] >= 0) {
            const float4 w4 = in[u] ? v[u] : make_float4(0.f, 0.f, 0.f, 0.f);
            D[at[u]] = w4.x; D[at[u] + 1] = w4.y; D[at[u] + 2] = w4.z; D[at[u] + 3] = w4.w;
          }
      }
    } else {
    for (int e0 = tid; e0 < nx; e0 += kThreads * kBatch) {
      float v[kBatch];
      int at[kBatch];
      bool in[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int e = e0 + u * kThreads;
        const int c = (int)__umulhi((unsigned)e, pl.chmagic), r2 = e - c * (PH * pl.XSg);
        const int pr = (int)__umulhi((unsigned)r2, pl.xsmagic), pc = r2 - pr * pl.XSg;
        const int h = h0 - a.pad + pr, w = w0 - a.pad + pc;
        in[u] = e < nx && c < a.C && pc < PW && h >= 0 && h < H && w >= 0 && w < W;
        at[u] = e < nx ? c * pl.XR + pr * pl.XS + pc : -1;
        const int cc = c < a.C ? c : a.C - 1;
        const int hc = h < 0 ? 0 : (h > H - 1 ? H - 1 : h), wc = w < 0 ? 0 : (w > W - 1 ? W - 1 : w);
        v[u] = xn[(size_t)cc * HW + (size_t)hc * W + wc];
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (at[u] >= 0) X[at[u]] = in[u] ? v[u] : 0.f;
    }
    for (int e0 = tid; e0 < nd; e0 += kThreads * kBatch) {
      float v[kBatch];
      bool in[kBatch];
      int at[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int e = e0 + u * kThreads;
        const int k = e >> pl.lgtile, r2 = e & ((1 << pl.lgtile) - 1);
        const int pr = r2 >> pl.lgTW, pc = r2 & (pl.TW - 1);
        const int h = h0 + pr, w = w0 + pc;
        at[u] = e < nd ? k * DK + pr * pl.DRS + pc : -1;
        in[u] = e < nd && k < a.T && h < H && w < W;
        const int kc = k < a.T ? k : a.T - 1, hc = h > H - 1 ? H - 1 : h, wc = w > W - 1 ? W - 1 : w;
        v[u] = dn[(size_t)kc * HW + (size_t)hc * W + wc];
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (at[u] >= 0) D[at[u]] = in[u] ? v[u] : 0.f;
    }
    }
    __syncthreads();
    // ---- this thread's runs: every S-th run of the tile ----
    if (active) {
      const int nruns = pl.TH * runs_per_row;
      for (int run = s; run < nruns; run += pl.S) {
        // Runs to lanes: in row-major order 16 lanes of a row would read cells L apart, a
        // few LDS banks only.  With `skew`, consecutive lanes take four runs of a row and then
        // the next row: rows are an odd number of cells apart, so 32 lanes (8 rows x 4 runs of
        // 8 cells) read 32 different banks.
        int row, col0;
        if (pl.skew) {
          const int quad = run >> 2;
          row = quad & (pl.TH - 1);
          col0 = (((quad >> (pl.lgtile - pl.lgTW)) << 2) + (run & 3)) * pl.L;
        } else {
          row = run / runs_per_row;
          col0 = (run - row * runs_per_row) * pl.L;
        }
        const float* xr = X + (size_t)(kCB * cb) * pl.XR + row * pl.XS + col0 + (pl.xlead - a.pad);
        const float* dr = D + (size_t)(KB * kb) * DK + row * pl.DRS + col0;
        // window columns col0 + t ... col0 + t + FS - 1; column (t + j) lives in slot (t + j) % FS
        float xw[kCB][FS][FS];
#pragma unroll
        for (int c = 0; c < kCB; ++c)
#pragma unroll
          for (int i = 0; i < FS; ++i)
#pragma unroll
            for (int j = 0; j + 1 < FS; ++j) xw[c][i][j] = xr[(size_t)c * pl.XR + i * pl.XS + j];
        for (int t0 = 0; t0 < pl.L; t0 += FS) {
#pragma unroll
          for (int tt = 0; tt < FS; ++tt) {
            const int tcol = t0 + tt;
            // (a run's length need not be a multiple of FS: steps past its end add zeros;
            //  the tile's rows have room for the reads)
            const bool live = tcol < pl.L;
#pragma unroll
            for (int c = 0; c < kCB; ++c)
#pragma unroll
              for (int i = 0; i < FS; ++i)
                xw[c][i][(tt + FS - 1) % FS] = xr[(size_t)c * pl.XR + i * pl.XS + tcol + FS - 1];
            float d[KB];
#pragma unroll
            for (int k = 0; k < KB; ++k) d[k] = live ? dr[(size_t)k * DK + tcol] : 0.f;
#pragma unroll
            for (int k = 0; k < KB; ++k)
#pragma unroll
              for (int c = 0; c < kCB; ++c)
#pragma unroll
                for (int i = 0; i < FS; ++i)
#pragma unroll
                  for (int j = 0; j < FS; ++j) acc[k][c][i][j] += d[k] * xw[c][i][(tt + j) % FS];
          }
        }
      }
    }
    __syncthreads();
  }
  // ---- sum over the S threads of a group, in order, through LDS; one partial set out ----
  // (as many groups at a time as the LDS holds: S sets of a thread's partial sums each)
  constexpr int kAcc = KB * kCB * FS * FS;
  float* red = lds;                                  // [group of the batch][S][kAcc]
  float* out = partial + (size_t)blockIdx.x * pl.outs;
  const int gbatch = pl.gbatch;
  for (int g0 = 0; g0 < pl.G; g0 += gbatch) {
    if (active && g >= g0 && g < g0 + gbatch) {
      float* mine = red + ((size_t)(g - g0) * pl.S + s) * kAcc;
      int o = 0;
#pragma unroll
      for (int k = 0; k < KB; ++k)
#pragma unroll
        for (int c = 0; c < kCB; ++c)
#pragma unroll
          for (int i = 0; i < FS; ++i)
#pragma unroll
            for (int j = 0; j < FS; ++j) mine[o++] = acc[k][c][i][j];
    }
    __syncthreads();
    const int ng = pl.G - g0 < gbatch ? pl.G - g0 : gbatch;
    for (int e = tid; e < ng * kAcc; e += kThreads) {
      const int gl = e / kAcc, o = e - gl * kAcc;
      const float* src = red + (size_t)gl * pl.S * kAcc + o;
      float sum = 0.f;
      for (int ss = 0; ss < pl.S; ++ss) sum += src[ss * kAcc];
      const int gg = g0 + gl, kbb = gg / pl.CBLK, cbb = gg - kbb * pl.CBLK;
      const int k = KB * kbb + o / (kCB * FS * FS), rem = o % (kCB * FS * FS);
      const int c = kCB * cbb + rem / (FS * FS), tap = rem % (FS * FS);
      if (k < a.T && c < a.C) out[((size_t)k * a.C + c) * (FS * FS) + tap] = sum;
    }
    __syncthreads();
  }
}

// ---- the same sums on the matrix cores, for more channels -------------------------------
// dK as a GEMM whose inner dimension is the pixels: rows = output channels k, columns
// n = (c, i, j), dK[k][n] = sum_p dy[k][p] * x[c][p + (i, j)], exact fp32 products from three
// bf16 parts per operand.  The LDS holds x (with its halo) and dy of a tile already split, as
// three planes of bf16 parts each (a tap's column reads the same x cells shifted: split per
// use, that work would be FS * FS times as much), in two buffers:
//   1. the next tile's cells are loaded into registers (four consecutive cells a thread and
//      slot; the cell a thread loads is the same in every tile, its offset worked out once);
//   2. the waves take their steps of 16 (32) consecutive pixels of a row of the current tile:
//      lane (k, part) reads its 8 pixels of dy[k] from the planes (16-byte reads), lane
//      (n, part) the 8 cells of column n's channel and tap (five dwords from the cell's even
//      neighbour on, shifted by 16 bits where it is odd); with 8 waves a block's reads are
//      issued before the block before it goes to the matrix cores;
//   3. the registers are split and written to the other buffer; one barrier per tile.
// A wave owns its accumulator blocks for the whole launch: `own` blocks of columns (every
// nbw-th) x MB blocks of output channels; the waves that share column blocks take every
// (waves / nbw)-th step and are added in fixed order at the end.  Two builds: 16 x 16 blocks
// (v_mfma_f32_16x16x32_bf16, steps of 32 pixels, up to eight blocks a wave) in workgroups of
// 16 waves for up to 32 output channels, and 32 x 32 blocks (v_mfma_f32_32x32x16_bf16, steps
// of 16 pixels, up to six blocks) in workgroups of 8 waves.  The first fits 128 registers, four
// waves per SIMD, which is what covers the latency of a block's chain (LDS reads -> shifts ->
// six dependent matrix instructions): N16 C16 K16 512x512 takes 205 us on it and 330 on the
// second (240 registers, two waves per SIMD), whose matrix-core time alone would be 124.
constexpr int kMThreads = 512, kMWaves = kMThreads / 64;
constexpr int kMaxAcc = 6;                   // 32 x 32 blocks a wave holds
constexpr int kMaxAcc16 = 8;                 // 16 x 16 blocks (up to 32 output channels, 16 waves)
constexpr int kMaxOuts = 16384;              // T * C * Y * X up to here
constexpr size_t kMLds = 160 * 1024;
constexpr int kSlots = 6;                    // groups of four cells a thread stages per tile

struct MfmaPlan {
  int TH, TW, lgTW, tilesX, tilesY, ntiles;
  int XS, XR, PHXS, DS;   // x: row stride, channel stride, cells of a channel's rows; dy: channel stride
  int vec, xlead;         // 16-byte loads; columns of x staged before the tile's first (pad, or 4)
  int nx, nd;             // cells staged: C * XR, T * DS (multiples of 4)
  int xplane, dplane;     // cells per plane (multiples of 8)
  int bufbytes;           // one buffer: three planes of x, three of dy
  int m16;                // up to 32 output channels: 16 x 16 blocks, steps of 32 pixels, 16 waves
  int NC, NB, MB;         // columns C * FS * FS; blocks of them; blocks of output channels
  int nbw, slices, own;   // waves across column blocks; waves across steps; column blocks a wave
  int rgroups;            // groups of waves across blocks of output channels (MB blocks each)
  int outs, grid;
  unsigned chmagic, xsmagic, dsmagic;
  size_t lds_bytes;
};

typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// One product of the split: 32 x 32 x 16 (lane: row or column lane % 32, eight of the 16
// pixels by lane / 32) or 16 x 16 x 32 (lane % 16, eight of 32 pixels by lane / 16).
__device__ __forceinline__ f32x16 mfma_any(u32x4 a, u32x4 b, f32x16 c) { return split::mfma16(a, b, c); }
__device__ __forceinline__ f32x4 mfma_any(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(split::bf16x8, a),
                                                 __builtin_bit_cast(split::bf16x8, b), c, 0, 0, 0);
}
template <class Acc>
__device__ __forceinline__ Acc mfma_split_any(u32x4 ah, u32x4 am, u32x4 al, u32x4 bh, u32x4 bm,
                                              u32x4 bl, Acc acc) {
  acc = mfma_any(al, bh, acc);
  acc = mfma_any(am, bm, acc);
  acc = mfma_any(ah, bl, acc);
  acc = mfma_any(am, bh, acc);
  acc = mfma_any(ah, bm, acc);
  acc = mfma_any(ah, bh, acc);
  return acc;
}
template <bool M16> struct AccOf { typedef f32x16 type; };
template <> struct AccOf<true> { typedef f32x4 type; };

__device__ __forceinline__ u32x4 funnel(const unsigned (&d)[5], unsigned shift) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = __builtin_amdgcn_alignbit(d[i + 1], d[i], shift);
  return r;
}
// Exact split of 4 floats into bf16 parts.
__device__ __forceinline__ void split4(const float (&v)[4], u32x2& h, u32x2& m, u32x2& l) {
#pragma unroll
  for (int d = 0; d < 2; ++d) {
    const float a = v[2 * d], b = v[2 * d + 1];
    h[d] = split::pack_hi16(a, b);
    const float ra = a - split::trunc_bf16(a), rb = b - split::trunc_bf16(b);
    m[d] = split::pack_hi16(ra, rb);
    const float sa = ra - split::trunc_bf16(ra), sb = rb - split::trunc_bf16(rb);
    l[d] = split::pack_hi16(sa, sb);
  }
}

template <int FS, int MB, bool M16>
__global__ __launch_bounds__(M16 ? 1024 : 512, M16 ? 4 : 2) void dense_mfma_kernel(BwdFilterArgs a, MfmaPlan pl,
                                                                  float* partial) {
  // blocks of BW x BW entries of dK, steps of 2^SPLG pixels, NV accumulator registers a block
  constexpr int BW = M16 ? 16 : 32, LGBW = M16 ? 4 : 5, SPLG = M16 ? 5 : 4, NV = M16 ? 4 : 16;
  constexpr int OWN = (M16 ? kMaxAcc16 : kMaxAcc) / MB;
  // threads: 16 waves where the accumulators are small (four waves per SIMD), else 8
  constexpr int THREADS = M16 ? 1024 : 512, SLOTS = kSlots * kMThreads / THREADS;
  typedef typename AccOf<M16>::type Acc;
  extern __shared__ float lds[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int l32 = lane & (BW - 1), hi = lane >> LGBW;   // row or column of a block; which eight pixels
  const int H = a.H, W = a.W, HW = H * W;
  // wave = (row group, step slice, column-block lane): a row group takes MB blocks of output
  // channels (more than MB blocks in all: two groups of waves, each with its own rows)
  const int b = wave & (pl.nbw - 1), rest = wave / pl.nbw;
  const int sl = rest % pl.slices, rg = rest / pl.slices;
  // this lane's column of every column block the wave owns, and its output channel of every
  // row block (past the last column / channel: the last one's cells, whose sums are not kept)
  int boff[OWN], aoff[MB];
#pragma unroll
  for (int o = 0; o < OWN; ++o) {
    int n = BW * (b + o * pl.nbw) + l32;
    n = n < pl.NC ? n : pl.NC - 1;
    const int c = n / (FS * FS), tap = n - c * (FS * FS), i = tap / FS, j = tap - i * FS;
    boff[o] = c * pl.XR + i * pl.XS + j + (pl.xlead - a.pad) + 8 * hi;
  }
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    int k = BW * (MB * rg + m) + l32;
    k = k < a.T ? k : a.T - 1;
    aoff[m] = k * pl.DS + 8 * hi;
  }
  // column blocks this wave has: b, b + nbw, ... below NB
  const int nown = (pl.NB - b + pl.nbw - 1) / pl.nbw;
  Acc acc[OWN][MB];
#pragma unroll
  for (int o = 0; o < OWN; ++o)
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
      for (int v = 0; v < NV; ++v) acc[o][m][v] = 0.f;

  // Slot q of this thread: the group of four cells g = tid + 512 q of the tile (x's groups,
  // then dy's): where it goes in the planes, its offset from the tile's first cell in memory,
  // and its row and column in the tile (-1: padding, zeros).
  const int xgroups = pl.nx >> 2, groups = xgroups + (pl.nd >> 2);
  unsigned rel[SLOTS];
  int rc[SLOTS];
#pragma unroll
  for (int q = 0; q < SLOTS; ++q) {
    const int g = tid + THREADS * q;
    if (g < xgroups) {
      const int e = 4 * g;
      const int c = (int)__umulhi((unsigned)e, pl.chmagic), r2 = e - c * pl.XR;
      const int pr = (int)__umulhi((unsigned)r2, pl.xsmagic), pc = r2 - pr * pl.XS;
      rel[q] = (unsigned)(c * HW + pr * W + pc);
      rc[q] = r2 < pl.PHXS ? (pr << 16) | pc : -1;
    } else {
      const int e = 4 * (g - xgroups);
      const int k = (int)__umulhi((unsigned)e, pl.dsmagic), r2 = e - k * pl.DS;
      const int pr = r2 >> pl.lgTW, pc = r2 & (pl.TW - 1);
      rel[q] = (unsigned)(k * HW + pr * W + pc);
      rc[q] = g < groups && pr < pl.TH ? (pr << 16) | pc : -1;
    }
  }

  const int tiles_per_image = pl.tilesX * pl.tilesY;
  const int lgcw = pl.lgTW - SPLG, nsteps = (pl.TH * pl.TW) >> SPLG;
  float4 held[SLOTS];
  // Tile t's cells into this thread's registers (zeros outside the image).
  auto fetch = [&](int t) {
    const int n = t / tiles_per_image, rem = t - n * tiles_per_image;
    const int ty = rem / pl.tilesX, tx = rem - ty * pl.tilesX;
    const int hx = ty * pl.TH - a.pad, wx = tx * pl.TW - pl.xlead;   // x's first staged cell
    const int hd = ty * pl.TH, wd = tx * pl.TW;                      // dy's
    const float* xn = a.x + (size_t)n * a.C * HW;
    const float* dn = a.dy + (size_t)n * a.T * HW;
#pragma unroll
    for (int q = 0; q < SLOTS; ++q) {
      const int g = tid + THREADS * q;
      const bool isx = g < xgroups;
      const int h0 = isx ? hx : hd, w0 = isx ? wx : wd;
      const float* src = isx ? xn : dn;
      const int h = h0 + (rc[q] >> 16), w = w0 + (rc[q] & 0xffff);
      const bool row_in = rc[q] >= 0 && (unsigned)h < (unsigned)H;
      const long at = (long)rel[q] + (long)h0 * W + w0;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (pl.vec) {
        // rows start at multiples of four columns and W % 4 == 0: four cells are inside
        // the image together or not at all
        if (row_in && (unsigned)w < (unsigned)W) v = *reinterpret_cast<const float4*>(src + at);
      } else if (row_in) {
        // (unaligned rows, or a width that four does not divide: cell by cell)
        if ((unsigned)w < (unsigned)W) v.x = src[at];
        if ((unsigned)(w + 1) < (unsigned)W) v.y = src[at + 1];
        if ((unsigned)(w + 2) < (unsigned)W) v.z = src[at + 2];
        if ((unsigned)(w + 3) < (unsigned)W) v.w = src[at + 3];
      }
      held[q] = v;
    }
  };
  // The registers, split, into buffer `buf`.
  auto deposit = [&](char* buf) {
#pragma unroll
    for (int q = 0; q < SLOTS; ++q) {
      const int g = tid + THREADS * q;
      if (g < groups) {
        const bool isx = g < xgroups;
        const int e = isx ? 4 * g : 4 * (g - xgroups);
        const int plane = isx ? pl.xplane : pl.dplane;
        char* base = buf + (isx ? 0 : 6 * pl.xplane) + 2 * e;
        const float v[4] = {held[q].x, held[q].y, held[q].z, held[q].w};
        u32x2 h, m, l;
        split4(v, h, m, l);
        *reinterpret_cast<u32x2*>(base) = h;
        *reinterpret_cast<u32x2*>(base + 2 * plane) = m;
        *reinterpret_cast<u32x2*>(base + 4 * plane) = l;
      }
    }
  };

  char* const bufs = reinterpret_cast<char*>(lds);
  const TileRange tr = tiles_of_workgroup(pl.ntiles);
  if (tr.first < tr.end) {
    fetch(tr.first);
    deposit(bufs);
  }
  __syncthreads();
  int it = 0;
  for (int t = tr.first; t < tr.end; t += tr.step, ++it) {
    const bool more = t + tr.step < tr.end;
    if (more) fetch(t + tr.step);
    const char* cur = bufs + (size_t)(it & 1) * pl.bufbytes;
    const unsigned* xp = reinterpret_cast<const unsigned*>(cur);
    const char* dp = cur + 6 * pl.xplane;
    const int xw = pl.xplane >> 1;                     // a plane of x in dwords
    // ---- this wave's steps ----
    for (int st = sl; st < nsteps; st += pl.slices) {
      const int row = st >> lgcw, col0 = (st & ((1 << lgcw) - 1)) << SPLG;
      u32x4 ah[MB], am[MB], al[MB];
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const char* p = dp + 2 * (aoff[m] + (row << pl.lgTW) + col0);
        ah[m] = *reinterpret_cast<const u32x4*>(p);
        am[m] = *reinterpret_cast<const u32x4*>(p + 2 * pl.dplane);
        al[m] = *reinterpret_cast<const u32x4*>(p + 4 * pl.dplane);
      }
      // cells off ... off + 7 of each plane: the dwords from off / 2, shifted by its parity
      // (row strides and steps are even: the parity is that of the lane's column)
      const int xo = row * pl.XS + col0;
      // (two sets of registers by the block's parity: a block's dwords are read while the
      //  block before it is in the matrix cores, and nothing is copied between the sets)
      if constexpr (!M16) {
        unsigned dh[2][5], dm[2][5], dl[2][5];
        {
          const unsigned* q = xp + ((boff[0] + xo) >> 1);
#pragma unroll
          for (int i = 0; i < 5; ++i) { dh[0][i] = q[i]; dm[0][i] = q[xw + i]; dl[0][i] = q[2 * xw + i]; }
        }
#pragma unroll
        for (int o = 0; o < OWN; ++o) {
          if (o < nown) {
            if (o + 1 < OWN && o + 1 < nown) {
              const unsigned* q = xp + ((boff[o + 1 < OWN ? o + 1 : o] + xo) >> 1);
#pragma unroll
              for (int i = 0; i < 5; ++i) {
                dh[(o + 1) & 1][i] = q[i]; dm[(o + 1) & 1][i] = q[xw + i]; dl[(o + 1) & 1][i] = q[2 * xw + i];
              }
            }
            const unsigned shift = (unsigned)(boff[o] & 1) * 16u;
            const u32x4 bh = funnel(dh[o & 1], shift), bm = funnel(dm[o & 1], shift), bl = funnel(dl[o & 1], shift);
#pragma unroll
            for (int m = 0; m < MB; ++m)
              acc[o][m] = mfma_split_any(ah[m], am[m], al[m], bh, bm, bl, acc[o][m]);
          }
        }
      } else {
        // (four waves per SIMD cover a block's reads; 128 registers leave no room for a second set)
#pragma unroll
        for (int o = 0; o < OWN; ++o) {
          if (o < nown) {
            const unsigned* q = xp + ((boff[o] + xo) >> 1);
            unsigned dh[5], dm[5], dl[5];
#pragma unroll
            for (int i = 0; i < 5; ++i) { dh[i] = q[i]; dm[i] = q[xw + i]; dl[i] = q[2 * xw + i]; }
            const unsigned shift = (unsigned)(boff[o] & 1) * 16u;
            const u32x4 bh = funnel(dh, shift), bm = funnel(dm, shift), bl = funnel(dl, shift);
#pragma unroll
            for (int m = 0; m < MB; ++m)
              acc[o][m] = mfma_split_any(ah[m], am[m], al[m], bh, bm, bl, acc[o][m]);
          }
        }
      }
    }
    if (more) deposit(bufs + (size_t)((it + 1) & 1) * pl.bufbytes);
    __syncthreads();
  }
  // ---- the waves that shared column blocks, added in order through LDS ----
  float* red = lds;                                  // [own block][row block][b][element][lane]
  for (int s2 = 1; s2 < pl.slices; ++s2) {
#pragma unroll
    for (int o = 0; o < OWN; ++o)
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        float* r = red + ((size_t)((rg * OWN + o) * MB + m) * pl.nbw + b) * (NV * 64) + lane;
        if (sl == s2 && o < pl.own) {
#pragma unroll
          for (int v = 0; v < NV; ++v) r[v << 6] = acc[o][m][v];
        }
      }
    __syncthreads();
#pragma unroll
    for (int o = 0; o < OWN; ++o)
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const float* r = red + ((size_t)((rg * OWN + o) * MB + m) * pl.nbw + b) * (NV * 64) + lane;
        if (sl == 0 && o < pl.own) {
#pragma unroll
          for (int v = 0; v < NV; ++v) acc[o][m][v] += r[v << 6];
        }
      }
    __syncthreads();
  }
  if (sl != 0) return;
  float* out = partial + (size_t)blockIdx.x * pl.outs;
#pragma unroll
  for (int o = 0; o < OWN; ++o) {
    const int n = BW * (b + o * pl.nbw) + l32;
    if (o < pl.own && n < pl.NC) {
#pragma unroll
      for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          // (accumulator element v: row 8 * (v / 4) + 4 * (lane / 32) + v % 4 of a 32 x 32 block,
          //  row 4 * (lane / 16) + v of a 16 x 16 one)
          const int k = M16 ? 16 * (MB * rg + m) + 4 * hi + v
                            : 32 * (MB * rg + m) + 8 * (v >> 2) + 4 * hi + (v & 3);
          if (k < a.T) out[(size_t)k * pl.NC + n] = acc[o][m][v];
        }
    }
  }
}

// dK[o] = sum over the partial sets in a fixed order: thread (o, y) adds sets y, y + LANES, ...,
// then the LANES partial sums are added in order through LDS (one thread summing all the sets
// of an entry would wait for several hundred loads one after the other).  Eight lanes of sets
// where dK has many entries, 32 where it has few (27 entries for three channels to one: a
// single workgroup, whose threads then wait for 24 loads each instead of 96).
constexpr int kRedOuts = 32;
template <int LANES>
__global__ __launch_bounds__(kRedOuts * LANES) void dense_reduce_kernel(const float* partial,
                                                                        float* dK, int outs,
                                                                        int sets) {
  __shared__ float part[LANES][kRedOuts];
  const int o = blockIdx.x * kRedOuts + threadIdx.x, y = threadIdx.y;
  float s = 0.f;
  if (o < outs) {
    int w = y;
    for (; w + 3 * LANES < sets; w += 4 * LANES) {
      const float v0 = partial[(size_t)w * outs + o];
      const float v1 = partial[(size_t)(w + LANES) * outs + o];
      const float v2 = partial[(size_t)(w + 2 * LANES) * outs + o];
      const float v3 = partial[(size_t)(w + 3 * LANES) * outs + o];
      s += v0;
      s += v1;
      s += v2;
      s += v3;
    }
    for (; w < sets; w += LANES) s += partial[(size_t)w * outs + o];
  }
  part[y][threadIdx.x] = s;
  __syncthreads();
  if (y == 0 && o < outs) {
    float t = part[0][threadIdx.x];
#pragma unroll
    for (int i = 1; i < LANES; ++i) t += part[i][threadIdx.x];
    dK[o] = t;
  }
}

// The chain rule from dK [T][C][Y][X] onto the factors.  A workgroup takes 32 ranks and one of
// the four gradients (blockIdx.y): dK and the factors' columns for those ranks go to LDS (read
// from memory inside the sums, every term would wait for a load of its own), then a thread
// takes a rank and every 32nd row of dFK or dFC, or, per output channel k, of the parts of
// dFH[i] or dFW[j], which are then added over k in order (a whole dFH row in one thread would
// be T * C * X terms long, the longest job by far).
constexpr int kFoldRanks = 32, kFoldRows = 32;
template <int FS>
__global__ __launch_bounds__(kFoldRanks * kFoldRows) void dense_fold_kernel(BwdFilterArgs a,
                                                                            const float* dK) {
  extern __shared__ float lds[];
  constexpr int Y = FS, X = FS;          // (square filters: the tap loops unroll, their loads overlap)
  const int T = a.T, C = a.C, R = a.R;
  const int outs = T * C * Y * X, frows = T + C + Y + X;
  float* dk = lds;                         // [T][C][Y][X]
  float* fac = lds + outs;                 // [T + C + Y + X][32]: FK, FC, FH, FW rows
  float* part = fac + frows * kFoldRanks;  // [FS][T][32]: per tap row or column and output channel
  const int tid = threadIdx.y * kFoldRanks + threadIdx.x;
  const int r0 = blockIdx.x * kFoldRanks, r = r0 + threadIdx.x;
  const int job = blockIdx.y;              // 0 dFK, 1 dFC, 2 dFH, 3 dFW
  // (dK in 16-byte pieces with four loads in flight a thread, the factors' columns with
  //  eight: one after the other, these loads were a third of the kernel's time)
  constexpr int kThreadsFold = kFoldRanks * kFoldRows;
  {
    const int quads = outs >> 2;
    const float4* src = reinterpret_cast<const float4*>(dK);
    float4* dst = reinterpret_cast<float4*>(dk);
    for (int e0 = tid; e0 < quads; e0 += 4 * kThreadsFold) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int e = e0 + u * kThreadsFold;
        v[u] = src[e < quads ? e : quads - 1];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (e0 + u * kThreadsFold < quads) dst[e0 + u * kThreadsFold] = v[u];
    }
    for (int e = 4 * quads + tid; e < outs; e += kThreadsFold) dk[e] = dK[e];
  }
  for (int e0 = tid; e0 < frows * kFoldRanks; e0 += 8 * kThreadsFold) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      int e = e0 + u * kThreadsFold;
      e = e < frows * kFoldRanks ? e : frows * kFoldRanks - 1;
      const int row = e / kFoldRanks, rr = r0 + (e % kFoldRanks);
      const float* src = row < T ? a.FK + (size_t)row * R
                       : row < T + C ? a.FC + (size_t)(row - T) * R
                       : row < T + C + Y ? a.FH + (size_t)(row - T - C) * R
                                         : a.FW + (size_t)(row - T - C - Y) * R;
      v[u] = src[rr < R ? rr : R - 1];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = e0 + u * kThreadsFold;
      if (e < frows * kFoldRanks) fac[e] = r0 + (e % kFoldRanks) < R ? v[u] : 0.f;
    }
  }
  __syncthreads();
  const float* fk = fac + threadIdx.x;                   // row stride kFoldRanks
  const float* fc = fk + T * kFoldRanks;
  const float* fh = fc + C * kFoldRanks;
  const float* fw = fh + Y * kFoldRanks;
  if (job == 0) {
    for (int k = threadIdx.y; k < T; k += kFoldRows) {
      float s = 0.f;
#pragma unroll 4
      for (int c = 0; c < C; ++c) {
        float sc = 0.f;
#pragma unroll
        for (int i = 0; i < Y; ++i) {
          float si = 0.f;
#pragma unroll
          for (int j = 0; j < X; ++j) si += dk[((k * C + c) * Y + i) * X + j] * fw[j * kFoldRanks];
          sc += si * fh[i * kFoldRanks];
        }
        s += sc * fc[c * kFoldRanks];
      }
      if (r < R) a.dFK[(size_t)k * R + r] = s;
    }
    return;
  }
  if (job == 1) {
    for (int c = threadIdx.y; c < C; c += kFoldRows) {
      float s = 0.f;
#pragma unroll 4
      for (int k = 0; k < T; ++k) {
        float sk = 0.f;
#pragma unroll
        for (int i = 0; i < Y; ++i) {
          float si = 0.f;
#pragma unroll
          for (int j = 0; j < X; ++j) si += dk[((k * C + c) * Y + i) * X + j] * fw[j * kFoldRanks];
          sk += si * fh[i * kFoldRanks];
        }
        s += sk * fk[k * kFoldRanks];
      }
      if (r < R) a.dFC[(size_t)c * R + r] = s;
    }
    return;
  }
  // the tap row i (dFH) or column j (dFW) and output channel k of q = i * T + k
  for (int q = threadIdx.y; q < FS * T; q += kFoldRows) {
    const int ij = q / T, k = q - ij * T;
    float s = 0.f;
#pragma unroll 4
    for (int c = 0; c < C; ++c) {
      float sc = 0.f;
      if (job == 2) {
#pragma unroll
        for (int j = 0; j < X; ++j) sc += dk[((k * C + c) * Y + ij) * X + j] * fw[j * kFoldRanks];
      } else {
#pragma unroll
        for (int i = 0; i < Y; ++i) sc += dk[((k * C + c) * Y + i) * X + ij] * fh[i * kFoldRanks];
      }
      s += sc * fc[c * kFoldRanks];
    }
    part[q * kFoldRanks + threadIdx.x] = s * fk[k * kFoldRanks];
  }
  __syncthreads();
  if (threadIdx.y < FS && r < R) {
    const float* p = part + (size_t)threadIdx.y * T * kFoldRanks + threadIdx.x;
    float s = 0.f;
    for (int k = 0; k < T; ++k) s += p[k * kFoldRanks];
    (job == 2 ? a.dFH : a.dFW)[(size_t)threadIdx.y * R + r] = s;
  }
}

size_t fold_lds_bytes(const cp4_shape& s) {
  return ((size_t)s.T * s.C * s.Y * s.X + (size_t)(s.T + s.C + s.Y + s.X) * kFoldRanks +
          (size_t)s.Y * s.T * kFoldRanks) * sizeof(float);
}

int kb_of(const cp4_shape& s) { return s.T >= 2 && s.Y <= 3 ? 2 : 1; }

bool plan(const cp4_shape& s, bool aligned16, DensePlan* best) {
  const int vec = aligned16 && s.W % 4 == 0 && s.W >= 4 ? 1 : 0, xlead = vec ? 4 : (int)s.pad;
  const int FS = (int)s.Y, KB = kb_of(s);
  const int KBLK = ((int)s.T + KB - 1) / KB, CBLK = ((int)s.C + kCB - 1) / kCB;
  const int G = KBLK * CBLK;
  if (G > kThreads) return false;
  int S = kThreads / G;                               // threads per group: a power of two
  while (S & (S - 1)) S &= S - 1;
  // (the sum over a group's threads goes through LDS, S sets of a thread's partial sums)
  while ((size_t)S * KB * kCB * FS * FS * sizeof(float) > kLdsLimit) S >>= 1;
  const int Cp = CBLK * kCB, Tp = KBLK * KB;
  const int cus = num_compute_units();
  bool found = false;
  double best_cost = 0;
  for (int TW = 32; TW <= 256; TW *= 2)
    for (int TH = 1; TH <= 32; TH *= 2) {
      // runs of L pixels, TH * TW / L of them over S threads; at least 8 pixels a run
      // where the tile allows, so that the sliding window pays
      int L = TW;
      while (L > 8 && (long)TH * TW / L < S) L >>= 1;
      // room for a run's last steps to read past it; with 16-byte loads the columns before
      // the tile's first, rows and channels multiples of four cells apart
      // (in LDS the rows of both tiles are an odd number of cells apart: lanes on consecutive
      //  rows then read different banks)
      const int XSg = vec ? (4 + TW + 2 * FS - 1 + 3) / 4 * 4 : TW + FS - 1 + FS;
      const int XS = XSg | 1, DRS = TW + 1;
      const int XR = (TH + FS - 1) * XS;
      const size_t lds = ((size_t)Cp * XR + (size_t)Tp * TH * DRS + FS) * sizeof(float);
      const size_t red = (size_t)S * KB * kCB * FS * FS * sizeof(float);
      if (lds > kLdsLimit || red > kLdsLimit) continue;
      DensePlan pl;
      pl.TH = TH; pl.TW = TW;
      pl.tilesX = ((int)s.W + TW - 1) / TW;
      pl.tilesY = ((int)s.H + TH - 1) / TH;
      pl.ntiles = (int)s.N * pl.tilesX * pl.tilesY;
      pl.KBLK = KBLK; pl.CBLK = CBLK; pl.G = G; pl.S = S; pl.L = L;
      pl.XS = XS; pl.XR = XR; pl.Cp = Cp; pl.Tp = Tp; pl.vec = vec; pl.xlead = xlead;
      pl.XSg = XSg; pl.DRS = DRS;
      pl.skew = (TW / L) % 4 == 0 && TH >= 2 ? 1 : 0;
      pl.outs = (int)(s.T * s.C * s.Y * s.X);
      pl.lgTW = __builtin_ctz(TW);
      pl.lgtile = __builtin_ctz(TW) + __builtin_ctz(TH);
      pl.chmagic = (unsigned)((0x100000000ull + (unsigned)((TH + FS - 1) * XSg) - 1) / (unsigned)((TH + FS - 1) * XSg));
      pl.xsmagic = (unsigned)((0x100000000ull + (unsigned)XSg - 1) / (unsigned)XSg);
      // workgroups per compute unit: what the LDS and the registers (two waves per SIMD with
      // two output channels a thread, three with one) leave room for
      const int by_lds = (int)(160 * 1024 / (lds > red ? lds : red));
      int per_cu = KB == 2 || FS >= 5 ? 2 : 3;
      per_cu = per_cu < by_lds ? per_cu : (by_lds < 1 ? 1 : by_lds);
      pl.grid = pl.ntiles < per_cu * cus ? pl.ntiles : per_cu * cus;
      if (pl.grid > kMaxGrid) pl.grid = kMaxGrid;
      {
        const size_t per_group = red;                 // S sets of a thread's partial sums
        size_t gb = kLdsLimit / per_group;
        gb = gb > (size_t)G ? (size_t)G : gb;
        pl.gbatch = (int)gb;
        const size_t all = gb * per_group;
        pl.lds_bytes = lds > all ? lds : all;
      }
      // cells moved per output pixel (halo, pixels past the image's edge), runs that leave
      // threads idle, and a grid that leaves compute units idle
      const double area = (double)pl.tilesX * TW * pl.tilesY * TH / ((double)s.W * s.H);
      const double halo = (double)(TH + FS - 1) * (TW + FS - 1) / ((double)TH * TW);
      const long nruns = (long)TH * TW / L;
      const double idle = (double)((nruns + S - 1) / S * S) / nruns;
      const double fill = (double)((pl.ntiles + pl.grid - 1) / pl.grid * pl.grid) / pl.ntiles;
      const double cost = area * (1.0 + 0.3 * halo) * idle * fill * (1.0 + 4.0 / L);
      if (!found || cost < best_cost) {
        best_cost = cost;
        *best = pl;
        found = true;
      }
    }
  return found;
}

template <int FS>
hipError_t launch_fs(const BwdFilterArgs& a, const DensePlan& pl, int kb, float* partial,
                     hipStream_t st) {
  if (kb == 2)
    dense_tiles_kernel<FS, 2><<<pl.grid, kThreads, pl.lds_bytes, st>>>(a, pl, partial);
  else
    dense_tiles_kernel<FS, 1><<<pl.grid, kThreads, pl.lds_bytes, st>>>(a, pl, partial);
  return hipGetLastError();
}

// LDS bank conflicts of a block's operand reads for a channel stride XR: the 32 lanes that the
// LDS serves together read dword (c * XR + i * XS + j + shift + 8 * part) / 2 of a plane, with
// (c, i, j) the lane's column of the GEMM; the worst number of different dwords on one of the 32
// banks, summed over the column blocks.
int read_conflicts(int XR, int XS, int FS, int NC, int shift, bool m16) {
  const int BW = m16 ? 16 : 32, NB = (NC + BW - 1) / BW;
  int total = 0;
  for (int nb = 0; nb < NB; ++nb) {
    int dwords[32];
    for (int l = 0; l < 32; ++l) {
      int n = BW * nb + (m16 ? (l & 15) : l);
      n = n < NC ? n : NC - 1;
      const int c = n / (FS * FS), tap = n - c * (FS * FS), i = tap / FS, j = tap - i * FS;
      dwords[l] = (c * XR + i * XS + j + shift + (m16 ? 8 * (l >> 4) : 0)) >> 1;
    }
    int count[32] = {0}, worst = 1;
    for (int l = 0; l < 32; ++l) {
      bool seen = false;
      for (int m = 0; m < l; ++m) seen = seen || dwords[m] == dwords[l];
      if (!seen && ++count[dwords[l] & 31] > worst) worst = count[dwords[l] & 31];
    }
    total += worst;
  }
  return total;
}

bool mfma_plan_blocks(const cp4_shape& s, bool aligned16, int m16, MfmaPlan* best) {
  const int vec = aligned16 && s.W % 4 == 0 ? 1 : 0, xlead = vec ? 4 : (int)s.pad;
  const int FS = (int)s.Y, T = (int)s.T, C = (int)s.C;
  const int BW = m16 ? 16 : 32, step = m16 ? 32 : 16;
  const int NC = C * FS * FS, NB = (NC + BW - 1) / BW, MBall = (T + BW - 1) / BW;
  // (a wave takes up to two blocks of output channels; with 16 x 16 blocks, 33 - 64 output
  //  channels go over two groups of waves)
  const int rgroups = MBall > 2 ? 2 : 1, MB = MBall > 2 ? 2 : MBall;
  if (MBall > 2 * rgroups || (!m16 && rgroups > 1) || (long)T * NC > kMaxOuts) return false;
  const int most_own = (m16 ? kMaxAcc16 : kMaxAcc) / MB;
  const int waves = (m16 ? 16 : kMWaves) / rgroups;   // per row group
  const int cus = num_compute_units();
  bool found = false;
  double best_cost = 0;
  // waves across the column blocks: as few as hold them all, or more (fewer waves then share
  // a tile's steps, which lets smaller tiles in where the LDS is short; groups of waves
  // without a block of their own idle)
  for (int nbw = 1; nbw <= waves; nbw *= 2) {
    if ((NB + nbw - 1) / nbw > most_own) continue;
    const int slices = waves / nbw, own = (NB + nbw - 1) / nbw;
    const size_t red = (size_t)rgroups * (m16 ? kMaxAcc16 : kMaxAcc) * nbw * (m16 ? 256 : 1024) * sizeof(float);
  for (int TW = step; TW <= 128; TW *= 2)
    for (int TH = 1; TH <= 32; TH *= 2) {
      if (TH * TW / step < slices) continue;
      const int PH = TH + FS - 1;
      // (a multiple of four: a group of four staged cells stays within a row)
      const int XS = vec ? TW + 8 : (TW + FS - 1 + 3) / 4 * 4;
      // a channel's rows (and up to 60 cells more, chosen below for the tile that wins)
      const int XR = (PH * XS + 3) / 4 * 4;
      const int DS = TH * TW + 8;                      // output channels four banks apart
      const int nx = C * XR, nd = T * DS;
      if ((nx + nd) / 4 > kSlots * kMThreads) continue;
      // LDS: two buffers of (x in three planes of bf16 parts | dy likewise); x's planes a few
      // cells longer: a column's reads end up to two cells past the last
      const int xplane = (nx + 8 + 7) / 8 * 8, dplane = (nd + 7) / 8 * 8;
      const int bufbytes = 6 * (xplane + dplane);
      size_t lds = 2 * (size_t)bufbytes;
      if (slices > 1 && red > lds) lds = red;
      if (lds > kMLds) continue;
      MfmaPlan pl;
      pl.TH = TH; pl.TW = TW;
      pl.lgTW = __builtin_ctz(TW);
      pl.tilesX = ((int)s.W + TW - 1) / TW;
      pl.tilesY = ((int)s.H + TH - 1) / TH;
      pl.ntiles = (int)s.N * pl.tilesX * pl.tilesY;
      pl.XS = XS; pl.XR = XR; pl.PHXS = PH * XS; pl.DS = DS; pl.vec = vec; pl.xlead = xlead;
      pl.nx = nx; pl.nd = nd; pl.xplane = xplane; pl.dplane = dplane; pl.bufbytes = bufbytes;
      pl.m16 = m16; pl.NC = NC; pl.NB = NB; pl.MB = MB;
      pl.nbw = nbw; pl.slices = slices; pl.own = own; pl.rgroups = rgroups;
      pl.outs = T * NC;
      pl.chmagic = (unsigned)((0x100000000ull + (unsigned)XR - 1) / (unsigned)XR);
      pl.xsmagic = (unsigned)((0x100000000ull + (unsigned)XS - 1) / (unsigned)XS);
      pl.dsmagic = (unsigned)((0x100000000ull + (unsigned)DS - 1) / (unsigned)DS);
      pl.lds_bytes = lds;
      pl.grid = pl.ntiles < cus ? pl.ntiles : cus;
      // (the partial sets stay within 24 MiB)
      const long set_bytes = ((long)pl.outs * 4 + 255) / 256 * 256;
      const long most = (24l << 20) / set_bytes - 1;
      if (pl.grid > most) pl.grid = (int)most;
      if (pl.grid > kMaxGrid) pl.grid = kMaxGrid;
      if (pl.grid < 1) continue;
      // cells staged per output pixel (halo, pixels past the image's edge), a grid that leaves
      // compute units idle, and the fixed cost of a tile
      const double area = (double)pl.tilesX * TW * pl.tilesY * TH / ((double)s.W * s.H);
      const double halo = (double)(PH * XS) / ((double)TH * TW);
      const double staged = ((double)C * halo + T) / (C + T);
      const double fill = (double)((pl.ntiles + pl.grid - 1) / pl.grid * pl.grid) / pl.ntiles;
      const double busy = (double)own * nbw / NB;      // (block slots per block)
      const double cost = area * fill * (0.5 + 0.5 * staged) * (1.0 + 64.0 / (TH * TW)) * busy;
      if (!found || cost < best_cost) {
        best_cost = cost;
        *best = pl;
        found = true;
      }
    }
  }
  if (!found) return false;
  // The channel stride of the winning tile: a channel's rows, then the few cells that leave
  // the operand reads with the fewest LDS bank conflicts (the taps of the channels that a
  // block's columns cover on different banks); what depends on it follows.
  MfmaPlan& pl = *best;
  const int XR0 = pl.XR;
  int fewest = 1 << 30;
  for (int cand = XR0; cand <= XR0 + 60; cand += 4) {
    const int nx = C * cand, xplane = (nx + 8 + 7) / 8 * 8;
    if ((nx + pl.nd) / 4 > kSlots * kMThreads || 12 * (size_t)(xplane + pl.dplane) > kMLds) break;
    const int cf = read_conflicts(cand, pl.XS, FS, NC, xlead - (int)s.pad, m16 != 0);
    if (cf < fewest) { fewest = cf; pl.XR = cand; }
  }
  pl.nx = C * pl.XR;
  pl.xplane = (pl.nx + 8 + 7) / 8 * 8;
  pl.bufbytes = 6 * (pl.xplane + pl.dplane);
  pl.lds_bytes = 2 * (size_t)pl.bufbytes;
  const size_t red = (size_t)rgroups * (m16 ? kMaxAcc16 : kMaxAcc) * pl.nbw * (m16 ? 256 : 1024) * sizeof(float);
  if (pl.slices > 1 && red > pl.lds_bytes) pl.lds_bytes = red;
  pl.chmagic = (unsigned)((0x100000000ull + (unsigned)pl.XR - 1) / (unsigned)pl.XR);
  return true;
}

// 16 x 16 blocks (all rows in use with up to 16 channels) on 16 waves, whose accumulators are
// small enough for four waves per SIMD (N16 C16 K16 512x512: 330 -> 204 us); where no tile of
// those fits, 32 x 32 blocks on 8 waves.
bool mfma_plan_uncached(const cp4_shape& s, bool aligned16, MfmaPlan* best) {
  if (mfma_plan_blocks(s, aligned16, 1, best)) return true;
  return mfma_plan_blocks(s, aligned16, 0, best);
}

// (the search above is tens of thousands of operations: the last few answers are kept per
//  thread; a layer's queries alternate between the two alignments and, with odd channel
//  counts, the layer's zero-padded shape)
bool mfma_plan(const cp4_shape& s, bool aligned16, MfmaPlan* best) {
  struct Entry {
    bool valid = false, aligned16 = false, found = false;
    cp4_shape shape;
    MfmaPlan plan;
  };
  constexpr int kEntries = 32;
  thread_local Entry cache[kEntries];
  thread_local int next = 0;
  for (int i = 0; i < kEntries; ++i) {
    const Entry& e = cache[i];
    if (e.valid && e.aligned16 == aligned16 && e.shape.N == s.N && e.shape.C == s.C &&
        e.shape.T == s.T && e.shape.H == s.H && e.shape.W == s.W && e.shape.pad == s.pad &&
        e.shape.Y == s.Y && e.shape.X == s.X && e.shape.Rank == s.Rank) {
      if (e.found) *best = e.plan;
      return e.found;
    }
  }
  Entry& e = cache[next];
  next = (next + 1) % kEntries;
  e.found = mfma_plan_uncached(s, aligned16, &e.plan);
  e.shape = s;
  e.aligned16 = aligned16;
  e.valid = true;
  if (e.found) *best = e.plan;
  return e.found;
}

template <int FS>
hipError_t launch_mfma_fs(const BwdFilterArgs& a, const MfmaPlan& pl, float* partial, hipStream_t st) {
  auto k0 = dense_mfma_kernel<FS, 1, true>;
  auto k02 = dense_mfma_kernel<FS, 2, true>;
  auto k1 = dense_mfma_kernel<FS, 1, false>;
  auto k2 = dense_mfma_kernel<FS, 2, false>;
  auto k = pl.m16 ? (pl.MB == 2 ? k02 : k0) : (pl.MB == 2 ? k2 : k1);
  if (pl.lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds_bytes);
    if (e != hipSuccess) return e;
  }
  k<<<pl.grid, pl.m16 ? 1024 : kMThreads, pl.lds_bytes, st>>>(a, pl, partial);
  return hipGetLastError();
}

template <int FS>
hipError_t launch_fold(const BwdFilterArgs& a, const float* dK, size_t lds, hipStream_t st) {
  auto k = dense_fold_kernel<FS>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
  }
  const dim3 fgrid((a.R + kFoldRanks - 1) / kFoldRanks, 4), fblock(kFoldRanks, kFoldRows);
  k<<<fgrid, fblock, lds, st>>>(a, dK);
  return hipGetLastError();
}

cp4_shape shape_of(const BwdFilterArgs& a) {
  cp4_shape s{};
  s.N = a.N; s.C = a.C; s.T = a.T; s.H = a.H; s.W = a.W; s.pad = a.pad; s.Y = a.Y; s.X = a.X; s.Rank = a.R;
  return s;
}

bool common_ok(const cp4_shape& s) {
  if (s.Y != s.X || !(s.Y == 1 || s.Y == 3 || s.Y == 5) || s.pad > s.Y - 1) return false;
  if (s.N == 0 || !fits_int_indexing((int)s.N, (int)s.H, (int)s.W)) return false;
  return fold_lds_bytes(s) <= 150 * 1024;
}

bool valu_ok(const cp4_shape& s) {
  DensePlan pl;
  return common_ok(s) && (long)s.T * s.C <= kMaxPairs && plan(s, false, &pl);
}

bool mfma_ok(const cp4_shape& s) {
  MfmaPlan pl;
  return common_ok(s) && mfma_plan(s, false, &pl);
}

// Which of the two tile kernels.  The matrix cores wherever they can run, except for one or
// two output channels under a 3x3 or 5x5 filter on large inputs: there a block of the GEMM is
// nearly empty and the plain multiply-adds are the faster ones (N128 C3 K1 512x512: 173 us
// against 360; N32 C16 K2 256x256: 79 against 97; N16 C16 K1 256x256 5x5: 85 against 124;
// but N32 C16 K3 256x256: 97 either way, N16 C16 K3 256x256 5x5: 175 against 128, and
// N8 C8 K2 256x256: 32 against 30).
std::atomic<int> g_forced_tile_kernel{-1};

bool use_mfma(const cp4_shape& s) {
  if (!mfma_ok(s)) return false;
  if (!valu_ok(s)) return true;
  const int forced = g_forced_tile_kernel.load();
  if (forced >= 0) return forced == 1;
  const double cells = (double)s.N * s.H * s.W * s.C;
  return !(s.T <= 2 && s.Y >= 3 && cells >= 1.0e7);
}

}  // namespace

bool bwd_filter_dense_tiles_supported(const cp4_shape& s) { return valu_ok(s) || mfma_ok(s); }

void bwd_filter_dense_tiles_force_kernel(int which) {
  g_forced_tile_kernel.store(which == 0 || which == 1 ? which : -1);
}

// Partial sets of the tile kernel, then the dense gradient itself.
size_t bwd_filter_dense_tiles_workspace_bytes(const cp4_shape& s) {
  const size_t set = ((size_t)s.T * s.C * s.Y * s.X * sizeof(float) + 255) / 256 * 256;
  size_t sets = 0;
  DensePlan dp;
  MfmaPlan mp;
  if (valu_ok(s) && plan(s, false, &dp)) sets = dp.grid;
  if (valu_ok(s) && plan(s, true, &dp) && (size_t)dp.grid > sets) sets = dp.grid;
  if (mfma_ok(s) && mfma_plan(s, false, &mp) && (size_t)mp.grid > sets) sets = mp.grid;
  if (mfma_ok(s) && mfma_plan(s, true, &mp) && (size_t)mp.grid > sets) sets = mp.grid;
  return (sets + 1) * set;
}

// Where this route is the faster one: linear time models (us) fitted by least squares to
// measured times of this route and of what the library runs without it, over 680 layers (1 -
// 64 channels a side, 1x1 / 3x3 / 5x5, ranks 4, 16 and 64, a thousand to a million pixels).
// With the matrix-core tile kernel: 14.9 us, 1.7 us per thousand entries of dK (the final
// sums and the chain rule), and per million pixels 0.68 us per channel staged and 8.8 per
// 32 x 32 block of the GEMM; without this route 17.6 us and per million pixels 116 us, 0.72
// per channel, 5.9 per rank and 0.1 per tap and rank where both channel counts are multiples
// of 16, and 25.2 us and 124, 0.37 (per channel of the counts rounded up to 16), 5.4 and 0.1
// where they run on zero-padded copies.  The smaller model picks the route: 0.3 % off the
// better one in the geometric mean (always this route 4 % off, never 96 %): it loses where
// both channel counts are multiples of 16 from 32 on under a 3x3 or 5x5 filter.
// With the plain multiply-add tile kernel: a fixed 18 us plus the final sums and the chain
// rule, and per million pixels the staging of the tiles (2.7 us per channel staged) and the
// multiply-adds (0.375 us per channel-block group and tap), against 26 us plus per million
// pixels 115 us and what grows with the planes.
// (N16 C16 K16 512x512 R16: 1040 us -> 215; N16 C3 K1 512x512 R16: 1005 -> 63; N8 C8 K8
// 256x256 R16: 132 -> 32; N16 C8 K8 256x256 R4: 210 -> 60; but N8 C32 K32 56x56 R16: 25
// against 33.)
bool bwd_filter_dense_tiles_preferred(const cp4_shape& s) {
  const double mpx = (double)s.N * s.H * s.W / 1.0e6;
  const double taps = (double)s.Y * s.X, macs = (double)s.T * s.C * taps;
  if (use_mfma(s)) {
    const double blocks = (double)((s.C * s.Y * s.X + 31) / 32) * ((s.T + 31) / 32);
    const double dense = 14.86 + 1.7325e-3 * macs +
                         mpx * (-4.73 + 0.6821 * (s.C + s.T) + 8.835 * blocks);
    // (channel counts that are multiples of 16 run as they are, others on zero-padded copies)
    const bool as_is = s.T % 16 == 0 && s.C % 16 == 0;
    const double padded = (double)((s.T + 15) / 16 * 16 + (s.C + 15) / 16 * 16);
    const double planes =
        as_is ? 17.64 + mpx * (115.6 + 0.7179 * padded + 5.944 * s.Rank + 0.0967 * taps * s.Rank)
              : 25.24 + mpx * (123.5 + 0.3736 * padded + 5.417 * s.Rank + 0.1013 * taps * s.Rank);
    return dense < planes;
  }
  const int kb = s.T >= 2 && s.Y <= 3 ? 2 : 1;
  const double groups = (double)((s.T + kb - 1) / kb) * ((s.C + kCB - 1) / kCB);
  const double staged = 1.2 * ((s.C + kCB - 1) / kCB * kCB) + s.T;
  const double dense = 18.0 + 0.05 * s.T * s.C + 0.008 * macs +
                       mpx * (-13.95 - 0.0232 * macs + 2.657 * staged + 0.3754 * groups * taps);
  const double planes = 25.79 + mpx * (1.371 * (s.T + s.C) - 0.3273 * s.Rank + 114.7 +
                                       0.2272 * taps * s.Rank);
  return dense < planes;
}

hipError_t bwd_filter_dense_tiles_launch(const BwdFilterArgs& a, hipStream_t st) {
  const cp4_shape s = shape_of(a);
  const int outs = a.T * a.C * a.Y * a.X;
  const size_t set = ((size_t)outs * sizeof(float) + 255) / 256 * 256 / sizeof(float);
  float* ws = static_cast<float*>(a.workspace);
  float* dK = ws;
  float* partial = ws + set;
  hipError_t e;
  int sets;
  // (the partial sets are `outs` apart; the padded stride is only what the size allows for)
  const bool aligned16 = ((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.dy)) & 15) == 0;
  if (use_mfma(s)) {
    MfmaPlan pl;
    if (!mfma_plan(s, aligned16, &pl) && !mfma_plan(s, false, &pl)) return hipErrorInvalidValue;
    sets = pl.grid;
    switch (a.Y) {
      case 1: e = launch_mfma_fs<1>(a, pl, partial, st); break;
      case 3: e = launch_mfma_fs<3>(a, pl, partial, st); break;
      default: e = launch_mfma_fs<5>(a, pl, partial, st); break;
    }
  } else {
    DensePlan pl;
    if (!valu_ok(s) || (!plan(s, aligned16, &pl) && !plan(s, false, &pl))) return hipErrorInvalidValue;
    sets = pl.grid;
    switch (a.Y) {
      case 1: e = launch_fs<1>(a, pl, kb_of(s), partial, st); break;
      case 3: e = launch_fs<3>(a, pl, kb_of(s), partial, st); break;
      default: e = launch_fs<5>(a, pl, kb_of(s), partial, st); break;
    }
  }
  if (e != hipSuccess) return e;
  if (outs <= 512)
    dense_reduce_kernel<32><<<(outs + kRedOuts - 1) / kRedOuts, dim3(kRedOuts, 32), 0, st>>>(
        partial, dK, outs, sets);
  else
    dense_reduce_kernel<8><<<(outs + kRedOuts - 1) / kRedOuts, dim3(kRedOuts, 8), 0, st>>>(
        partial, dK, outs, sets);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  const size_t fold_lds = fold_lds_bytes(s);
  switch (a.Y) {
    case 1: return launch_fold<1>(a, dK, fold_lds, st);
    case 3: return launch_fold<3>(a, dK, fold_lds, st);
    default: return launch_fold<5>(a, dK, fold_lds, st);
  }
}

}  // namespace cp4
