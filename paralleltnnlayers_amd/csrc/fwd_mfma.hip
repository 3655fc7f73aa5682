// Fused forward / backward-data kernel on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32) for ranks up to 64.
//
// One workgroup (8 wave64) owns a strip of TH image rows of one image, full
// width.  Each channel plane of a strip plus its halo rows is one contiguous
// run of floats in NCHW, so pixels are handled as a flat index q.
//
//   P0  Fin[Cin,R] -> LDS, zero-padded to RP = 32*RB columns.
//   P1  A[r,q] = sum_c Fin[c,r] x[c,q] for the strip + halo rows.  Each wave
//       owns blocks of 64 consecutive pixels; a lane streams float2 (two
//       pixels) per channel straight from HBM into registers, double-buffered
//       kPF channel pairs deep, and feeds them as the B operand of the MFMA;
//       the A operand is 64 consecutive floats of the LDS copy of Fin.  The
//       accumulators go to LDS as A[r][q]; rows outside the image become 0.
//   P2  taps along H (A -> B) then along W (B -> Cc), VALU out of LDS, the
//       rank index wave-uniform so the tap weights are scalar operands.
//   P3  y[k,p] = sum_r Fout[k,r] Cc[r,p]: a wave keeps the Fout fragment of
//       its 32-output-channel block in registers, reads Cc pairs from LDS as
//       the B operand and stores float2 per lane, 256 contiguous bytes per
//       half-wave and output row.
//
// x is read once from HBM (halo rows are shared with the neighbouring strip,
// which the XCD-aware tile order places on the same L2), y is written once,
// and no intermediate leaves the CU.  Arithmetic follows the reassociated form
// of Cuda_kernels/cp4Conv2dForward.cu:84-133 (backward-data:
// cp4Conv2dBackwardData.cu:57-108 through swapped factors and flipped taps).
#include "cp4_internal.h"

namespace cp4 {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 512, kWaves = kThreads / 64;
constexpr int kPF = 8;                       // channel pairs per prefetch chunk
constexpr size_t kLdsLimit = 160 * 1024;     // gfx950 LDS per workgroup

struct StripPlan {
  int TH;       // output rows per strip
  int strips;   // strips per image
  int nWG;      // N * strips
  int QA;       // LDS row stride of A / Cc (floats)
  int QB;       // LDS row stride of B (floats)
  int padoff;   // leading floats of each B row (>= pad, even)
  size_t lds_bytes;
};

__device__ __forceinline__ f32x16 mfma32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

template <int RB>
__global__ __launch_bounds__(kThreads) void fwd_mfma_strip_kernel(FwdArgs a, StripPlan pl) {
  constexpr int RP = 32 * RB;
  extern __shared__ float lds[];
  float* As = lds;                 // [RP][QA]: A after P1, Cc after P2
  float* R2 = lds + RP * pl.QA;    // Fin tile [Cin][RP] in P1, B [RP][QB] in P2

  // XCD-aware tile order: workgroup b runs on XCD b % 8; give each XCD a
  // contiguous range of tiles so neighbouring strips share an L2.
  const int per = (pl.nWG + 7) >> 3;
  const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (t >= pl.nWG) return;
  const int n = t / pl.strips, h0 = (t - n * pl.strips) * pl.TH;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;
  const int H = a.H, W = a.W, HW = H * W, R = a.R, Cin = a.Cin, Cout = a.Cout;
  const int QA = pl.QA, QB = pl.QB;

  // ---- P0: input-channel factor to LDS -----------------------------------
  for (int i = tid; i < Cin * RP; i += kThreads) {
    const int c = i / RP, r = i - c * RP;
    R2[i] = r < R ? a.Fin[(size_t)c * R + r] : 0.f;
  }
  __syncthreads();

  // ---- P1: channel -> rank contraction -----------------------------------
  const int qbase = (h0 - a.pad) * W;          // global flat pixel of LDS column 0
  const int QLEN = (pl.TH + a.Y - 1) * W;
  const int npair = (QLEN + 63) >> 6;
  const float* xn = a.x + (size_t)n * Cin * HW;
  const int nsteps = Cin >> 1;                 // channel pairs
  const int nchunks = nsteps / kPF;

  for (int pb = wave; pb < npair; pb += kWaves) {
    const int qa = pb * 64 + 2 * l32;
    const int q = qbase + qa;
    const bool valid = q >= 0 && q < HW && qa < QLEN;
    f32x16 acc[RB][2];
#pragma unroll
    for (int mb = 0; mb < RB; ++mb) {
      acc[mb][0] = (f32x16)(0.f);
      acc[mb][1] = (f32x16)(0.f);
    }
    if (__any(valid)) {
      const int qc = q < 0 ? 0 : (q > HW - 2 ? HW - 2 : q);
      const float* xp = xn + (size_t)hi * HW + qc;   // channel (2*step + hi)
      const float* fp = R2 + hi * RP + l32;           // Fin[2*step + hi][32*mb + l32]
      float2 xb0[kPF], xb1[kPF];

      auto load = [&](float2 (&xb)[kPF], int ch) {
#pragma unroll
        for (int s = 0; s < kPF; ++s)
          xb[s] = *reinterpret_cast<const float2*>(xp + (size_t)(2 * (ch * kPF + s)) * HW);
      };
      auto compute = [&](const float2 (&xb)[kPF], int ch) {
#pragma unroll
        for (int s = 0; s < kPF; ++s) {
          const float* f = fp + (ch * kPF + s) * 2 * RP;
#pragma unroll
          for (int mb = 0; mb < RB; ++mb) {
            const float aop = f[32 * mb];
            acc[mb][0] = mfma32(aop, xb[s].x, acc[mb][0]);
            acc[mb][1] = mfma32(aop, xb[s].y, acc[mb][1]);
          }
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
      for (int st = nchunks * kPF; st < nsteps; ++st) {   // channel-pair remainder
        const float2 xv = *reinterpret_cast<const float2*>(xp + (size_t)(2 * st) * HW);
        const float* f = fp + st * 2 * RP;
#pragma unroll
        for (int mb = 0; mb < RB; ++mb) {
          const float aop = f[32 * mb];
          acc[mb][0] = mfma32(aop, xv.x, acc[mb][0]);
          acc[mb][1] = mfma32(aop, xv.y, acc[mb][1]);
        }
      }
    }
    // accumulator (v, lane) holds rank row 8*(v/4) + 4*hi + v%4, pixel column l32
#pragma unroll
    for (int mb = 0; mb < RB; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = 32 * mb + 8 * (v >> 2) + 4 * hi + (v & 3);
        float2 o;
        o.x = valid ? acc[mb][0][v] : 0.f;
        o.y = valid ? acc[mb][1][v] : 0.f;
        *reinterpret_cast<float2*>(As + r * QA + qa) = o;
      }
  }
  __syncthreads();

  // ---- P2: taps along H, then along W ------------------------------------
  const int npix = pl.TH * W;   // output pixels of a full strip
  float* Bs = R2 + pl.padoff;
  for (int rr = wave; rr < RP; rr += kWaves) {
    const float* ar = As + rr * QA;
    float* br = Bs + rr * QB;
    if (rr < R) {
      for (int p = lane; p < npix; p += 64) {
        float s = 0.f;
        for (int i = 0; i < a.Y; ++i)
          s += a.FH[(a.flip ? a.Y - 1 - i : i) * R + rr] * ar[p + i * W];
        br[p] = s;
      }
    }
  }
  __syncthreads();
  for (int p = lane; p < npix; p += 64) {
    const int w = p % W;
    for (int rr = wave; rr < RP; rr += kWaves) {
      const float* br = Bs + rr * QB;
      float s = 0.f;
      if (rr < R) {
        for (int j = 0; j < a.X; ++j) {
          const int ww = w + j - a.pad;
          const float bv = (ww >= 0 && ww < W) ? br[p + j - a.pad] : 0.f;
          s += a.FW[(a.flip ? a.X - 1 - j : j) * R + rr] * bv;
        }
      }
      As[rr * QA + p] = s;
    }
  }
  __syncthreads();

  // ---- P3: rank -> output-channel contraction ----------------------------
  const int rows = min(pl.TH, H - h0);
  const int nvalid = rows * W;
  const int npo = (nvalid + 63) >> 6;
  const int nkb = (Cout + 31) >> 5;
  float* yn = a.y + (size_t)n * Cout * HW + (size_t)h0 * W;
  float fk[RP / 2];
  int cur_kb = -1;
  for (int item = wave; item < nkb * npo; item += kWaves) {
    const int pp = item / nkb, kb = item - pp * nkb;
    if (kb != cur_kb) {
      cur_kb = kb;
      const int k = 32 * kb + l32;
#pragma unroll
      for (int s = 0; s < RP / 2; ++s) {
        const int r = 2 * s + hi;
        fk[s] = (k < Cout && r < R) ? a.Fout[(size_t)k * R + r] : 0.f;
      }
    }
    f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
    const float* cp = As + hi * QA + pp * 64 + 2 * l32;
#pragma unroll
    for (int s = 0; s < RP / 2; ++s) {
      const float2 b = *reinterpret_cast<const float2*>(cp + 2 * s * QA);
      acc0 = mfma32(fk[s], b.x, acc0);
      acc1 = mfma32(fk[s], b.y, acc1);
    }
    const int p = pp * 64 + 2 * l32;
    if (p < nvalid) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int k = 32 * kb + 8 * (v >> 2) + 4 * hi + (v & 3);
        if (k < Cout) {
          float2 o;
          o.x = acc0[v];
          o.y = acc1[v];
          *reinterpret_cast<float2*>(yn + (size_t)k * HW + p) = o;
        }
      }
    }
  }
}

int round_up(int v, int m) { return (v + m - 1) / m * m; }

// LDS layout for a strip height; returns false if it does not fit.
bool layout(const FwdArgs& a, int TH, StripPlan* pl) {
  const int RP = a.R <= 32 ? 32 : 64;
  const long QLEN = (long)(TH + a.Y - 1) * a.W;
  const long QA = round_up((int)QLEN, 64) + 8;
  const int padoff = round_up(a.pad, 2);
  const long QB = round_up(TH * a.W + padoff + a.X, 2);
  const long r2 = (long)a.Cin * RP > RP * QB ? (long)a.Cin * RP : RP * QB;
  const size_t bytes = (size_t)(RP * QA + r2) * sizeof(float);
  if (bytes > kLdsLimit) return false;
  pl->TH = TH;
  pl->strips = (a.H + TH - 1) / TH;
  pl->nWG = a.N * pl->strips;
  pl->QA = (int)QA;
  pl->QB = (int)QB;
  pl->padoff = padoff;
  pl->lds_bytes = bytes;
  return true;
}

// Strip height: fewest rounds of 256 workgroups times the per-strip matrix work
// (halo rows repeat the channel->rank contraction).
bool plan(const FwdArgs& a, StripPlan* best) {
  double best_cost = 0;
  bool found = false;
  for (int TH = 1; TH <= a.H; ++TH) {
    StripPlan pl;
    if (!layout(a, TH, &pl)) break;
    const double rounds = (pl.nWG + 255) / 256;
    const double cost = rounds * ((double)(TH + a.Y - 1) * a.Cin + (double)TH * a.Cout);
    if (!found || cost < best_cost) {
      best_cost = cost;
      *best = pl;
      found = true;
    }
  }
  return found;
}

}  // namespace

bool fwd_mfma_supported(const FwdArgs& a) {
  if (a.R > 64 || (a.W & 1) || (a.Cin & 1)) return false;
  if (a.x && (reinterpret_cast<uintptr_t>(a.x) & 7)) return false;
  if (a.y && (reinterpret_cast<uintptr_t>(a.y) & 7)) return false;
  StripPlan pl;
  return plan(a, &pl);
}

hipError_t fwd_mfma_launch(const FwdArgs& a, hipStream_t st) {
  StripPlan pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
  const unsigned grid = 8u * ((pl.nWG + 7) / 8);
  hipError_t e;
  if (a.R <= 32) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(fwd_mfma_strip_kernel<1>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds_bytes);
    if (e != hipSuccess) return e;
    fwd_mfma_strip_kernel<1><<<grid, kThreads, pl.lds_bytes, st>>>(a, pl);
  } else {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(fwd_mfma_strip_kernel<2>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds_bytes);
    if (e != hipSuccess) return e;
    fwd_mfma_strip_kernel<2><<<grid, kThreads, pl.lds_bytes, st>>>(a, pl);
  }
  return hipGetLastError();
}

}  // namespace cp4
