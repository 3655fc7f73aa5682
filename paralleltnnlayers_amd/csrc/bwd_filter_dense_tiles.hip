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
//   1. dense_tiles_kernel<FS, KB>: persistent workgroups of 256 threads over tiles of
//      TH x TW pixels; the x tile with its halo and the dy tile go to LDS (zero outside the
//      image); a thread owns KB output channels x 4 input channels x FS x FS taps in
//      registers and a run of consecutive pixels of one row, along which the FS x FS window of
//      x slides (FS new cells per channel and pixel); partial sums stay in registers across a
//      workgroup's tiles, are added over the threads that share a channel block through LDS in
//      fixed order, and leave as one partial set per workgroup.
//   2. dense_reduce_kernel: the partial sets summed in fixed order.
//   3. dense_fold_kernel: the chain rule, one thread per factor-gradient entry.
// No atomics: bit-reproducible.  Plain fp32 multiply-adds.
#include "cp4_internal.h"

namespace cp4 {
namespace {

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
  int XS, XR;          // x tile in LDS: row stride, rows * XS per channel (padded)
  int Cp, Tp;          // channel counts padded to their blocks
  int outs;            // T * C * FS * FS
  int lgTW, lgtile;    // log2 of TW and of TH * TW
  unsigned chmagic;    // ceil(2^32 / ((TH + FS - 1) * XS))
  unsigned xsmagic;    // ceil(2^32 / XS)
  int gbatch;          // groups whose partial sums the LDS holds at a time in the final sum
  int grid;
  size_t lds_bytes;
};

template <int FS, int KB>
__global__ __launch_bounds__(kThreads) void dense_tiles_kernel(BwdFilterArgs a, DensePlan pl,
                                                               float* partial) {
  extern __shared__ float lds[];
  float* X = lds;                                    // [Cp][TH + FS - 1][XS]
  float* D = lds + (size_t)pl.Cp * pl.XR;            // [Tp][TH][TW]
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

  const int tiles_per_image = pl.tilesX * pl.tilesY;
  for (int t = blockIdx.x; t < pl.ntiles; t += gridDim.x) {
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
    const int nx = pl.Cp * PH * pl.XS;
    for (int e0 = tid; e0 < nx; e0 += kThreads * kBatch) {
      float v[kBatch];
      int at[kBatch];
      bool in[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int e = e0 + u * kThreads;
        const int c = (int)__umulhi((unsigned)e, pl.chmagic), r2 = e - c * (PH * pl.XS);
        const int pr = (int)__umulhi((unsigned)r2, pl.xsmagic), pc = r2 - pr * pl.XS;
        const int h = h0 - a.pad + pr, w = w0 - a.pad + pc;
        in[u] = e < nx && c < a.C && pc < PW && h >= 0 && h < H && w >= 0 && w < W;
        at[u] = e < nx ? c * pl.XR + r2 : -1;
        const int cc = c < a.C ? c : a.C - 1;
        const int hc = h < 0 ? 0 : (h > H - 1 ? H - 1 : h), wc = w < 0 ? 0 : (w > W - 1 ? W - 1 : w);
        v[u] = xn[(size_t)cc * HW + (size_t)hc * W + wc];
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (at[u] >= 0) X[at[u]] = in[u] ? v[u] : 0.f;
    }
    const float* dn = a.dy + (size_t)n * a.T * HW;
    const int nd = pl.Tp * pl.TH * pl.TW;
    for (int e0 = tid; e0 < nd; e0 += kThreads * kBatch) {
      float v[kBatch];
      bool in[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int e = e0 + u * kThreads;
        const int k = e >> pl.lgtile, r2 = e & ((1 << pl.lgtile) - 1);
        const int pr = r2 >> pl.lgTW, pc = r2 & (pl.TW - 1);
        const int h = h0 + pr, w = w0 + pc;
        in[u] = e < nd && k < a.T && h < H && w < W;
        const int kc = k < a.T ? k : a.T - 1, hc = h > H - 1 ? H - 1 : h, wc = w > W - 1 ? W - 1 : w;
        v[u] = dn[(size_t)kc * HW + (size_t)hc * W + wc];
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (e0 + u * kThreads < nd) D[e0 + u * kThreads] = in[u] ? v[u] : 0.f;
    }
    __syncthreads();
    // ---- this thread's runs: every S-th run of the tile ----
    if (active) {
      const int nruns = pl.TH * runs_per_row;
      for (int run = s; run < nruns; run += pl.S) {
        const int row = run / runs_per_row, col0 = (run - row * runs_per_row) * pl.L;
        const float* xr = X + (size_t)(kCB * cb) * pl.XR + row * pl.XS + col0;
        const float* dr = D + (size_t)(KB * kb) * pl.TH * pl.TW + row * pl.TW + col0;
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
            for (int k = 0; k < KB; ++k) d[k] = live ? dr[(size_t)k * pl.TH * pl.TW + tcol] : 0.f;
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

// dK[o] = sum over the partial sets in a fixed order: thread (o, y) adds sets y, y + 8, ...,
// then the eight partial sums are added in order through LDS (one thread summing all the sets
// of an entry would wait for several hundred loads one after the other).
constexpr int kRedOuts = 32, kRedSets = 8;
__global__ __launch_bounds__(kRedOuts * kRedSets) void dense_reduce_kernel(const float* partial,
                                                                           float* dK, int outs,
                                                                           int sets) {
  __shared__ float part[kRedSets][kRedOuts];
  const int o = blockIdx.x * kRedOuts + threadIdx.x, y = threadIdx.y;
  float s = 0.f;
  if (o < outs) {
    int w = y;
    for (; w + 3 * kRedSets < sets; w += 4 * kRedSets) {
      const float v0 = partial[(size_t)w * outs + o];
      const float v1 = partial[(size_t)(w + kRedSets) * outs + o];
      const float v2 = partial[(size_t)(w + 2 * kRedSets) * outs + o];
      const float v3 = partial[(size_t)(w + 3 * kRedSets) * outs + o];
      s += v0;
      s += v1;
      s += v2;
      s += v3;
    }
    for (; w < sets; w += kRedSets) s += partial[(size_t)w * outs + o];
  }
  part[y][threadIdx.x] = s;
  __syncthreads();
  if (y == 0 && o < outs) {
    float t = part[0][threadIdx.x];
#pragma unroll
    for (int i = 1; i < kRedSets; ++i) t += part[i][threadIdx.x];
    dK[o] = t;
  }
}

// The chain rule from dK [T][C][Y][X] onto the factors.  A workgroup takes 32 ranks: dK and
// the factors' columns for those ranks go to LDS (read from memory inside the sums, every term
// would wait for a load of its own), then a thread takes (rank, every 32nd row of the four
// gradients).
constexpr int kFoldRanks = 32, kFoldRows = 32;
template <int FS>
__global__ __launch_bounds__(kFoldRanks * kFoldRows) void dense_fold_kernel(BwdFilterArgs a,
                                                                            const float* dK) {
  extern __shared__ float lds[];
  constexpr int Y = FS, X = FS;          // (square filters: the tap loops unroll, their loads overlap)
  const int T = a.T, C = a.C, R = a.R;
  const int outs = T * C * Y * X, rows = T + C + Y + X;
  float* dk = lds;                         // [T][C][Y][X]
  float* fac = lds + outs;                 // [T + C + Y + X][32]: FK, FC, FH, FW rows
  const int tid = threadIdx.y * kFoldRanks + threadIdx.x;
  const int r0 = blockIdx.x * kFoldRanks, r = r0 + threadIdx.x;
  for (int e = tid; e < outs; e += kFoldRanks * kFoldRows) dk[e] = dK[e];
  for (int e = tid; e < rows * kFoldRanks; e += kFoldRanks * kFoldRows) {
    const int row = e / kFoldRanks, rr = r0 + (e % kFoldRanks);
    const float* src = row < T ? a.FK + (size_t)row * R
                     : row < T + C ? a.FC + (size_t)(row - T) * R
                     : row < T + C + Y ? a.FH + (size_t)(row - T - C) * R
                                       : a.FW + (size_t)(row - T - C - Y) * R;
    fac[e] = rr < R ? src[rr] : 0.f;
  }
  __syncthreads();
  const float* fk = fac + threadIdx.x;                   // row stride kFoldRanks
  const float* fc = fk + T * kFoldRanks;
  const float* fh = fc + C * kFoldRanks;
  const float* fw = fh + Y * kFoldRanks;
  if (r >= R) return;
  for (int row = threadIdx.y; row < rows; row += kFoldRows) {
    float s = 0.f;
    if (row < T) {
      const int k = row;
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
      a.dFK[(size_t)k * R + r] = s;
    } else if (row < T + C) {
      const int c = row - T;
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
      a.dFC[(size_t)c * R + r] = s;
    } else if (row < T + C + Y) {
      const int i = row - T - C;
      for (int k = 0; k < T; ++k) {
        float sk = 0.f;
#pragma unroll 4
        for (int c = 0; c < C; ++c) {
          float sc = 0.f;
#pragma unroll
          for (int j = 0; j < X; ++j) sc += dk[((k * C + c) * Y + i) * X + j] * fw[j * kFoldRanks];
          sk += sc * fc[c * kFoldRanks];
        }
        s += sk * fk[k * kFoldRanks];
      }
      a.dFH[(size_t)i * R + r] = s;
    } else {
      const int j = row - T - C - Y;
      for (int k = 0; k < T; ++k) {
        float sk = 0.f;
#pragma unroll 4
        for (int c = 0; c < C; ++c) {
          float sc = 0.f;
#pragma unroll
          for (int i = 0; i < Y; ++i) sc += dk[((k * C + c) * Y + i) * X + j] * fh[i * kFoldRanks];
          sk += sc * fc[c * kFoldRanks];
        }
        s += sk * fk[k * kFoldRanks];
      }
      a.dFW[(size_t)j * R + r] = s;
    }
  }
}

int kb_of(const cp4_shape& s) { return s.T >= 2 && s.Y <= 3 ? 2 : 1; }

bool plan(const cp4_shape& s, DensePlan* best) {
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
      const int XS = TW + FS - 1 + FS;                // room for a run's last steps to read past it
      const int XR = (TH + FS - 1) * XS + 1;          // odd-ish channel stride against bank conflicts
      const size_t lds = ((size_t)Cp * XR + (size_t)Tp * TH * TW + FS) * sizeof(float);
      const size_t red = (size_t)S * KB * kCB * FS * FS * sizeof(float);
      if (lds > kLdsLimit || red > kLdsLimit) continue;
      DensePlan pl;
      pl.TH = TH; pl.TW = TW;
      pl.tilesX = ((int)s.W + TW - 1) / TW;
      pl.tilesY = ((int)s.H + TH - 1) / TH;
      pl.ntiles = (int)s.N * pl.tilesX * pl.tilesY;
      pl.KBLK = KBLK; pl.CBLK = CBLK; pl.G = G; pl.S = S; pl.L = L;
      pl.XS = XS; pl.XR = XR; pl.Cp = Cp; pl.Tp = Tp;
      pl.outs = (int)(s.T * s.C * s.Y * s.X);
      pl.lgTW = __builtin_ctz(TW);
      pl.lgtile = __builtin_ctz(TW) + __builtin_ctz(TH);
      pl.chmagic = (unsigned)((0x100000000ull + (unsigned)((TH + FS - 1) * XS) - 1) / (unsigned)((TH + FS - 1) * XS));
      pl.xsmagic = (unsigned)((0x100000000ull + (unsigned)XS - 1) / (unsigned)XS);
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

}  // namespace

bool bwd_filter_dense_tiles_supported(const cp4_shape& s) {
  if (s.Y != s.X || !(s.Y == 1 || s.Y == 3 || s.Y == 5) || s.pad > s.Y - 1) return false;
  if ((long)s.T * s.C > kMaxPairs || s.N == 0) return false;
  if (!fits_int_indexing((int)s.N, (int)s.H, (int)s.W)) return false;
  DensePlan pl;
  return plan(s, &pl);
}

// Partial sets of the tile kernel, then the dense gradient itself.
size_t bwd_filter_dense_tiles_workspace_bytes(const cp4_shape& s) {
  const size_t outs = (size_t)s.T * s.C * s.Y * s.X;
  return (kMaxGrid + 1) * ((outs * sizeof(float) + 255) / 256 * 256);
}

// Where this route is the faster one: two linear time models (us) fitted by least squares to
// both routes over 378 layers (3 - 32 channels a side, 1x1 / 3x3 / 5x5, ranks 4 and 16, a
// thousand to a million pixels; the choice they make is 3 % off the better route in the
// geometric mean).  Here a fixed 18 us plus the final sums and the chain rule (0.05 us per
// channel pair, 0.008 per multiply-add of a pixel, M = T * C * Y * X), and per million pixels the staging of the tiles (2.7 us per
// channel staged) and the multiply-adds (0.375 us per channel-block group and tap); the
// factor-by-factor variants 26 us plus per million pixels 115 us and what grows with the
// planes (N16 C3 K1 512x512 R16: 1005 us -> 63; N8 C8 K8 256x256 R16: 132 -> 52; N16 C16 K16
// 512x512 R16: 1058 -> 900; but N1 C16 K16 32x32 R8: 21 against 54).
bool bwd_filter_dense_tiles_preferred(const cp4_shape& s) {
  const double mpx = (double)s.N * s.H * s.W / 1.0e6;
  const double taps = (double)s.Y * s.X, macs = (double)s.T * s.C * taps;
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
  cp4_shape s{};
  s.N = a.N; s.C = a.C; s.T = a.T; s.H = a.H; s.W = a.W; s.pad = a.pad; s.Y = a.Y; s.X = a.X; s.Rank = a.R;
  DensePlan pl;
  if (!plan(s, &pl)) return hipErrorInvalidValue;
  const size_t set = ((size_t)pl.outs * sizeof(float) + 255) / 256 * 256 / sizeof(float);
  float* ws = static_cast<float*>(a.workspace);
  float* dK = ws;
  float* partial = ws + set;
  hipError_t e;
  // (the partial sets are pl.outs apart; the padded stride is only what the size allows for)
  switch (a.Y) {
    case 1: e = launch_fs<1>(a, pl, kb_of(s), partial, st); break;
    case 3: e = launch_fs<3>(a, pl, kb_of(s), partial, st); break;
    default: e = launch_fs<5>(a, pl, kb_of(s), partial, st); break;
  }
  if (e != hipSuccess) return e;
  dense_reduce_kernel<<<(pl.outs + kRedOuts - 1) / kRedOuts, dim3(kRedOuts, kRedSets), 0, st>>>(
      partial, dK, pl.outs, pl.grid);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  const size_t fold_lds = ((size_t)pl.outs + (size_t)(a.T + a.C + a.Y + a.X) * kFoldRanks) * sizeof(float);
  const dim3 fgrid((a.R + kFoldRanks - 1) / kFoldRanks), fblock(kFoldRanks, kFoldRows);
  switch (a.Y) {
    case 1: dense_fold_kernel<1><<<fgrid, fblock, fold_lds, st>>>(a, dK); break;
    case 3: dense_fold_kernel<3><<<fgrid, fblock, fold_lds, st>>>(a, dK); break;
    default: dense_fold_kernel<5><<<fgrid, fblock, fold_lds, st>>>(a, dK); break;
  }
  return hipGetLastError();
}

}  // namespace cp4
