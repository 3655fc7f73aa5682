// Forward / backward-data for layers with very few channels on both sides
// (3 -> 1, say): the cheaper association of the same sum.
//
// The CP4 operator is y[k] = sum_{c,i,j} K[k,c,i,j] x[c,h+i-p,w+j-p] with
// K[k,c,i,j] = sum_r Fout[k,r] Fin[c,r] FH[i,r] FW[j,r]
// (Cuda_kernels/cp4Conv2dForward.cu:84-133 sums the same terms; Utils.cu:55-62 is
// this K).  The factor-by-factor order costs R*(Cin + Y + X + Cout) multiply-adds
// per pixel, the recomposed order Cout*Cin*Y*X: with three channels in, one out
// and a 3x3 filter that is 27 against 160 at rank 16, and the pass becomes
// bound by memory instead of by the vector units.  The caller picks this kernel
// only where the recomposed order is the cheaper one.
//
// One workgroup (256 threads) owns `tpw` vertically adjacent tiles of 16 rows x
// 64 columns of one image and up to eight output channels (more output channels:
// more workgroups).  With FwdArgs::dense the filter K is given instead of the
// factors (the reshaped-CP sibling op recomposes its own); a given filter of any
// number of input channels is taken - beyond 8192 weights per workgroup only the
// current channel chunk's weights are in LDS, reloaded with every chunk:
//   prologue  the four factors go to LDS, then every workgroup recomposes K into
//             LDS itself (Cout*Cin*Y*X*R multiply-adds: a few thousand, no scratch
//             memory, no extra launch; the tiles of a workgroup share it)
//   per tile and chunk of input channels: the tile plus halo goes to LDS,
//             zero-padded outside the image (one float4 per lane for the 64 inner
//             columns where alignment allows); a thread owns four neighbouring
//             columns of one row and all output channels, reads the FS + 3 cells
//             of a filter row once and uses each for up to four pixels; weights
//             are LDS broadcasts
//   epilogue  one float4 store per output channel where alignment allows
// Tap order follows FwdArgs::flip (backward-data reads the taps in reverse,
// Cuda_kernels/cp4Conv2dBackwardData.cu:79-87).
#include "cp4_internal.h"

namespace cp4 {
namespace {

constexpr int kTH = 16, kTW = 64, kPX = 4, kThreads = 256;
constexpr int kMaxWeights = 8192;             // floats of recomposed filter in LDS
constexpr int kMaxFactorFloats = 8192;        // the four factors, staged in the tile's LDS
constexpr size_t kTileBudget = 96 * 1024;     // bytes of LDS for the input tile

struct DensePlan {
  int cc;        // input channels per chunk
  int tile_w;    // LDS row length of the tile (floats, odd: conflict-free segment reads)
  int tpw;       // tiles per workgroup, down the image
  int wfloats;   // LDS floats set aside for a workgroup's filter (a multiple of 4)
  int stream_w;  // the filter does not fit: only the current channel chunk's weights are
                 // in LDS, reloaded with every chunk of the tile (given filters only)
  int cols, rowgroups, ntiles;   // tile columns, groups of tpw tile rows, workgroups with work
  size_t lds_bytes;
};

// SW: the filter does not fit LDS and streams by channel chunk (DensePlan::stream_w).
template <int FS, int KO, bool SW>
__global__ __launch_bounds__(kThreads) void fwd_dense_small_kernel(FwdArgs a, DensePlan pl) {
  extern __shared__ float lds[];
  const int Cin = a.Cin, R = a.R, H = a.H, W = a.W;
  // Workgroup b runs on XCD b % 8, each with an L2 of its own: tile ids are permuted
  // so that an XCD gets a contiguous range - horizontally adjacent tiles, which
  // share their halo columns' cache lines, then meet in one L2 (with the plain
  // x-fastest grid the kernel fetched 2.1 times its input).
  const int per = (pl.ntiles + 7) >> 3;
  const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (t >= pl.ntiles) return;                         // whole workgroup, before any barrier
  const int bx = t % pl.cols, by = (t / pl.cols) % pl.rowgroups, bz = t / (pl.cols * pl.rowgroups);
  // output channels in groups of eight, one group per workgroup (bz = image, group)
  const int ngrp = (a.Cout + 7) >> 3;
  const int n = bz / ngrp, k0 = 8 * (bz - n * ngrp);
  const int Cout = min(8, a.Cout - k0);               // channels of this group
  const int nw = Cout * Cin * FS * FS;
  float* wts = lds;                                   // [Cout][Cin][FS][FS]
  float* tile = lds + pl.wfloats;                     // [cc][kTH + FS - 1][tile_w]
  const int tid = threadIdx.x;
  const int w0 = bx * kTW;
  const size_t HW = (size_t)H * W;

  if (a.dense) {
    // the filter is given: [Cout][Cin][FS][FS], taps in the order this pass reads them
    if (!SW) {
      const float* src = a.dense + (size_t)k0 * Cin * FS * FS;
      for (int q = tid; q < nw; q += kThreads) wts[q] = src[q];
    }
  } else {
    // the factors once through LDS (they alias the tile, which is loaded later) ...
    float* fo = tile;                                 // Fout [Cout][R]
    float* fi = fo + Cout * R;                        // Fin  [Cin][R]
    float* fh = fi + Cin * R;                         // FH   [FS][R]
    float* fw = fh + FS * R;                          // FW   [FS][R]
    for (int q = tid; q < Cout * R; q += kThreads) fo[q] = a.Fout[(size_t)k0 * R + q];
    for (int q = tid; q < Cin * R; q += kThreads) fi[q] = a.Fin[q];
    for (int q = tid; q < FS * R; q += kThreads) {
      fh[q] = a.FH[q];
      fw[q] = a.FW[q];
    }
    __syncthreads();
    // ... and the recomposed filter, taps already in the order this pass reads them
    for (int q = tid; q < nw; q += kThreads) {
      const int j = q % FS, i = (q / FS) % FS, c = (q / (FS * FS)) % Cin, k = q / (FS * FS * Cin);
      const int ti = a.flip ? FS - 1 - i : i, tj = a.flip ? FS - 1 - j : j;
      const float *p0 = fo + k * R, *p1 = fi + c * R, *p2 = fh + ti * R, *p3 = fw + tj * R;
      float s = 0.f;
      for (int r = 0; r < R; ++r) s += p0[r] * p1[r] * p2[r] * p3[r];
      wts[q] = s;
    }
  }

  constexpr int kUnrollI = FS <= 5 ? FS : 1;         // filter rows unrolled only for small filters
  constexpr int HT = kTH + FS - 1, WC = kTW + FS - 1; // rows and cells per row of tile + halo
  const int ty = tid >> 4, tx = tid & 15;             // row of the tile, group of four columns
  const int WT = pl.tile_w;
  const int left = a.pad;                             // halo cells left of the tile (pad <= FS - 1)
  const bool vec_in = (W & 3) == 0 && w0 + kTW <= W && (reinterpret_cast<uintptr_t>(a.x) & 15) == 0;
  const bool vec_out = (W & 3) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 15) == 0;
  const float* xn = a.x + (size_t)n * Cin * HW;

  for (int tr = 0; tr < pl.tpw; ++tr) {
    const int h0 = (by * pl.tpw + tr) * kTH;
    if (h0 >= H) break;
    float acc[KO][kPX];
#pragma unroll
    for (int k = 0; k < KO; ++k)
#pragma unroll
      for (int p = 0; p < kPX; ++p) acc[k][p] = 0.f;

    for (int c0 = 0; c0 < Cin; c0 += pl.cc) {
      const int cn = min(pl.cc, Cin - c0);
      __syncthreads();                                // weights written / previous tile read
      const int nrows = cn * HT;                      // (channel, tile row) pairs
      if (SW) {
        // this chunk's weights: [Cout][cn][FS][FS] out of the filter's [Cout][Cin][FS][FS]
        const int per = cn * FS * FS;
        for (int q = tid; q < Cout * per; q += kThreads) {
          const int k = q / per, e = q - k * per;
          wts[q] = a.dense[((size_t)(k0 + k) * Cin + c0) * FS * FS + e];
        }
      }
      if (vec_in) {
        // the 64 inner columns of a row: sixteen float4
        for (int q = tid; q < nrows * 16; q += kThreads) {
          const int rowid = q >> 4, v = q & 15;
          const int c = rowid / HT, row = rowid - c * HT;
          const int gh = h0 + row - a.pad;
          float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
          if (gh >= 0 && gh < H)
            val = *reinterpret_cast<const float4*>(xn + (size_t)(c0 + c) * HW + (size_t)gh * W + w0 + 4 * v);
          float* dst = tile + rowid * WT + left + 4 * v;
          dst[0] = val.x;
          dst[1] = val.y;
          dst[2] = val.z;
          dst[3] = val.w;
        }
        // the FS - 1 halo columns of a row
        constexpr int kHalo = FS > 1 ? FS - 1 : 1;    // (FS == 1: the loop below is empty)
        for (int q = tid; q < nrows * (FS - 1); q += kThreads) {
          const int rowid = q / kHalo, e = q - rowid * kHalo;
          const int c = rowid / HT, row = rowid - c * HT;
          const int col = e < left ? e : kTW + e;     // cell of the row: left halo, then right halo
          const int gh = h0 + row - a.pad, gw = w0 + col - left;
          float v = 0.f;
          if (gh >= 0 && gh < H && gw >= 0 && gw < W) v = xn[(size_t)(c0 + c) * HW + (size_t)gh * W + gw];
          tile[rowid * WT + col] = v;
        }
      } else {
        for (int q = tid; q < nrows * WC; q += kThreads) {
          const int rowid = q / WC, col = q - rowid * WC;
          const int c = rowid / HT, row = rowid - c * HT;
          const int gh = h0 + row - a.pad, gw = w0 + col - left;
          float v = 0.f;
          if (gh >= 0 && gh < H && gw >= 0 && gw < W) v = xn[(size_t)(c0 + c) * HW + (size_t)gh * W + gw];
          tile[rowid * WT + col] = v;
        }
      }
      __syncthreads();
      for (int c = 0; c < cn; ++c) {
#pragma unroll kUnrollI
        for (int i = 0; i < FS; ++i) {
          float seg[kPX + FS - 1];
          const float* src = tile + (c * HT + ty + i) * WT + kPX * tx;
#pragma unroll
          for (int e = 0; e < kPX + FS - 1; ++e) seg[e] = src[e];
#pragma unroll
          for (int k = 0; k < KO; ++k) {
            if (k < Cout) {
              const float* wr = SW ? wts + ((k * cn + c) * FS + i) * FS
                                            : wts + ((k * Cin + c0 + c) * FS + i) * FS;
#pragma unroll
              for (int j = 0; j < FS; ++j) {
                const float wv = wr[j];
#pragma unroll
                for (int p = 0; p < kPX; ++p) acc[k][p] += wv * seg[p + j];
              }
            }
          }
        }
      }
    }

    const int h = h0 + ty, w = w0 + kPX * tx;
    if (h < H && w < W) {
      float* yp = a.y + ((size_t)n * a.Cout + k0) * HW + (size_t)h * W + w;
      const bool vec = vec_out && w + kPX <= W;
#pragma unroll
      for (int k = 0; k < KO; ++k) {
        if (k < Cout) {
          float* dst = yp + (size_t)k * HW;
          // y = act(conv + bias[k]) as the values are stored (FwdArgs::bias / act)
          const float bk = a.bias ? a.bias[k0 + k] : 0.f;
          float o[kPX];
#pragma unroll
          for (int p = 0; p < kPX; ++p) {
            const float t = acc[k][p] + bk;
            o[p] = (a.act != 0 && t < 0.f) ? 0.f : t;
          }
          if (vec) {
            *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
          } else {
#pragma unroll
            for (int p = 0; p < kPX; ++p)
              if (w + p < W) dst[p] = o[p];
          }
        }
      }
    }
  }
}

bool plan(const FwdArgs& a, DensePlan* pl) {
  if (a.Y != a.X || !(a.Y & 1) || a.Y > 17 || a.pad > a.Y - 1) return false;
  if (a.ldf || a.accumulate || a.sh) return false;
  const int kgrp = a.Cout < 8 ? a.Cout : 8;           // output channels of a workgroup
  const long ngrp = (a.Cout + 7) / 8;
  long nw = (long)kgrp * a.Cin * a.Y * a.X;
  const bool stream_w = nw > kMaxWeights;
  if (stream_w && (!a.dense || (long)kgrp * a.Y * a.X > kMaxWeights)) return false;
  const long nf = a.dense ? 0 : (long)a.R * (kgrp + a.Cin + a.Y + a.X);
  if (nf > kMaxFactorFloats) return false;

  // odd row length: the four-column segments of neighbouring threads fall on
  // different LDS banks
  const int tile_w = (kTW + a.Y - 1) | 1;
  const size_t per_channel = (size_t)(kTH + a.Y - 1) * tile_w * sizeof(float);
  int cc = (int)(kTileBudget / per_channel);
  if (cc < 1) return false;
  if (cc > a.Cin) cc = a.Cin;
  if (stream_w) {
    const int wcc = (int)(kMaxWeights / ((long)kgrp * a.Y * a.X));   // channels whose weights fit
    if (cc > wcc) cc = wcc;
    nw = (long)kgrp * cc * a.Y * a.X;
  }
  size_t tile_bytes = cc * per_channel;
  if (tile_bytes < (size_t)nf * sizeof(float)) tile_bytes = (size_t)nf * sizeof(float);
  // enough workgroups to fill the device sixteen times over, each amortising its
  // filter recomposition over several tiles
  const long row_tiles = (a.H + kTH - 1) / kTH, col_tiles = (a.W + kTW - 1) / kTW;
  const long tiles = row_tiles * col_tiles * a.N * ngrp;
  long tpw = tiles / (16l * num_compute_units());
  if (tpw < 1) tpw = 1;
  if (tpw > row_tiles) tpw = row_tiles;
  if (tpw > 16) tpw = 16;
  const long rowgroups = (row_tiles + tpw - 1) / tpw;
  const long ntiles = col_tiles * rowgroups * a.N * ngrp;
  if (ntiles > (1l << 30)) return false;
  pl->cols = (int)col_tiles;
  pl->rowgroups = (int)rowgroups;
  pl->ntiles = (int)ntiles;
  pl->cc = cc;
  pl->tile_w = tile_w;
  pl->tpw = (int)tpw;
  pl->wfloats = (int)((nw + 3) & ~3l);
  pl->stream_w = stream_w ? 1 : 0;
  pl->lds_bytes = (size_t)pl->wfloats * sizeof(float) + tile_bytes;
  return true;
}

template <int FS, int KO, bool SW>
hipError_t launch_sw(const FwdArgs& a, const DensePlan& pl, hipStream_t st) {
  const void* fn = reinterpret_cast<const void*>(fwd_dense_small_kernel<FS, KO, SW>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds_bytes);
  if (e != hipSuccess) return e;
  const unsigned grid = 8u * ((pl.ntiles + 7) / 8);
  fwd_dense_small_kernel<FS, KO, SW><<<grid, kThreads, pl.lds_bytes, st>>>(a, pl);
  return hipGetLastError();
}
template <int FS, int KO>
hipError_t launch_as(const FwdArgs& a, const DensePlan& pl, hipStream_t st) {
  return pl.stream_w ? launch_sw<FS, KO, true>(a, pl, st) : launch_sw<FS, KO, false>(a, pl, st);
}

template <int FS>
hipError_t launch_ko(const FwdArgs& a, const DensePlan& pl, hipStream_t st) {
  if (a.Cout <= 1) return launch_as<FS, 1>(a, pl, st);
  if (a.Cout <= 2) return launch_as<FS, 2>(a, pl, st);
  if (a.Cout <= 4) return launch_as<FS, 4>(a, pl, st);
  return launch_as<FS, 8>(a, pl, st);              // groups of eight, the last one may be short
}

}  // namespace

bool fwd_dense_small_supported(const FwdArgs& a) {
  DensePlan pl;
  return plan(a, &pl);
}

bool fwd_dense_small_plan_info(const FwdArgs& a, long* tiles, size_t* lds_bytes) {
  DensePlan pl;
  if (!plan(a, &pl)) return false;
  *tiles = (long)pl.ntiles * pl.tpw;
  *lds_bytes = pl.lds_bytes;
  return true;
}

hipError_t fwd_dense_small_launch(const FwdArgs& a, hipStream_t st) {
  DensePlan pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
  switch (a.Y) {
    case 1: return launch_ko<1>(a, pl, st);
    case 3: return launch_ko<3>(a, pl, st);
    case 5: return launch_ko<5>(a, pl, st);
    case 7: return launch_ko<7>(a, pl, st);
    case 9: return launch_ko<9>(a, pl, st);
    case 11: return launch_ko<11>(a, pl, st);
    case 13: return launch_ko<13>(a, pl, st);
    case 15: return launch_ko<15>(a, pl, st);
    default: return launch_ko<17>(a, pl, st);
  }
}

}  // namespace cp4
