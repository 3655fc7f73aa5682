// General forward / backward-data kernel: any rank, channel counts, odd or
// even filter size, pad, stride and output size; VALU arithmetic, LDS-tiled.
//
// One workgroup owns an 8 x 32 output tile of one image and walks the rank in
// blocks of RB.  Per rank block:
//   1. A[r][halo pixel] = sum_c Fin[c,r] x[c, pixel]   (global -> registers -> LDS;
//      32 consecutive lanes read 32 consecutive floats of one NCHW row)
//   2. B[r][h][halo col] = sum_i FH[i,r] A[r][h+i][col]          (LDS -> LDS)
//   3. Cc[r] = sum_j FW[j,r] B[r][h][w+j]                        (LDS -> registers)
//   4. y[k, pixel] (+)= sum_r Fout[k,r] Cc[r]                    (registers -> global)
// Factor values are wave-uniform and come through scalar loads.  The
// arithmetic is the reassociated form of Cuda_kernels/cp4Conv2dForward.cu:84-133:
// the spatial taps are applied to R rank planes instead of C channel planes.
#include "cp4_internal.h"

namespace cp4 {
namespace {

constexpr int kTH = 8, kTW = 32, kThreads = kTH * kTW;

template <int RB>
__global__ __launch_bounds__(kThreads) void fwd_general_kernel(FwdArgs a, Geometry g) {
  extern __shared__ float lds[];
  // input cells under a tile of kTH x kTW outputs: rows, columns
  const int HT = g.sh * (kTH - 1) + a.Y, WT = g.sw * (kTW - 1) + a.X;
  const int nA = HT * WT, nB = kTH * WT;
  float* As = lds;            // [RB][HT*WT]
  float* Bs = lds + RB * nA;  // [RB][kTH*WT]
  const int n = blockIdx.z, h0 = blockIdx.y * kTH, w0 = blockIdx.x * kTW;   // output coordinates
  const int tid = threadIdx.x;
  const size_t HW = (size_t)a.H * a.W, HWo = (size_t)g.Ho * g.Wo;
  const float* xn = a.x + (size_t)n * a.Cin * HW;
  const int R = a.R;

  for (int r0 = 0; r0 < R; r0 += RB) {
    // 1. channel -> rank contraction on the halo tile
    for (int q = tid; q < nA; q += kThreads) {
      const int hh = q / WT, ww = q - hh * WT;
      const int gh = g.sh * h0 + hh - g.pt, gw = g.sw * w0 + ww - g.pl;
      float acc[RB];
#pragma unroll
      for (int rr = 0; rr < RB; ++rr) acc[rr] = 0.f;
      if (gh >= 0 && gh < a.H && gw >= 0 && gw < a.W) {
        const float* xp = xn + (size_t)gh * a.W + gw;
#pragma unroll 4
        for (int c = 0; c < a.Cin; ++c) {     // (unrolled: the scalar factor loads of four channels overlap)
          const float v = xp[c * HW];
          const float* f = a.Fin + (size_t)c * R + r0;
#pragma unroll
          for (int rr = 0; rr < RB; ++rr)
            acc[rr] += v * (r0 + rr < R ? f[rr] : 0.f);
        }
      }
#pragma unroll
      for (int rr = 0; rr < RB; ++rr) As[rr * nA + q] = acc[rr];
    }
    __syncthreads();
    // 2. taps along H
    for (int q = tid; q < nB; q += kThreads) {
      const int h = q / WT, ww = q - h * WT;
#pragma unroll
      for (int rr = 0; rr < RB; ++rr) {
        float s = 0.f;
        if (r0 + rr < R)
          for (int i = 0; i < a.Y; ++i)
            s += a.FH[(a.flip ? a.Y - 1 - i : i) * R + r0 + rr] *
                 As[rr * nA + (g.sh * h + i) * WT + ww];
        Bs[rr * nB + q] = s;
      }
    }
    __syncthreads();
    // 3. taps along W, one output pixel per thread
    const int h = tid / kTW, w = tid - h * kTW;
    float cc[RB];
#pragma unroll
    for (int rr = 0; rr < RB; ++rr) {
      float s = 0.f;
      if (r0 + rr < R)
        for (int j = 0; j < a.X; ++j)
          s += a.FW[(a.flip ? a.X - 1 - j : j) * R + r0 + rr] *
               Bs[rr * nB + h * WT + g.sw * w + j];
      cc[rr] = s;
    }
    // 4. rank -> output-channel contraction
    if (h0 + h < g.Ho && w0 + w < g.Wo) {
      float* yp = a.y + (size_t)n * a.Cout * HWo + (size_t)(h0 + h) * g.Wo + w0 + w;
#pragma unroll 4
      for (int k = 0; k < a.Cout; ++k) {      // (unrolled: four rows of the factor in flight)
        const float* f = a.Fout + (size_t)k * R + r0;
        float s = 0.f;
#pragma unroll
        for (int rr = 0; rr < RB; ++rr) s += cc[rr] * (r0 + rr < R ? f[rr] : 0.f);
        if (r0 > 0) s += yp[k * HWo];
        yp[k * HWo] = s;
      }
    }
    __syncthreads();
  }
}

// LDS floats needed for a rank block of rb.
size_t lds_floats(const FwdArgs& a, int rb) {
  const Geometry g = geometry_of(a);
  const size_t HT = (size_t)g.sh * (kTH - 1) + a.Y, WT = (size_t)g.sw * (kTW - 1) + a.X;
  return (size_t)rb * (HT * WT + kTH * WT);
}
// More LDS per workgroup costs occupancy, a second rank block re-reads and
// re-writes y: with many output channels the second costs more (N1 C3 K96
// 224x224 11x11 R16: 80 us in one block of 70 KB, 99 us in two), with few the
// first (N1 C3 K1 512x512 17x17 R16: 239 against 126 us).
constexpr size_t kLdsBudget = 64 * 1024, kLdsBudgetManyOutputs = 96 * 1024;
constexpr int kManyOutputs = 32;

int pick_rank_block(const FwdArgs& a) {
  const size_t budget = a.Cout >= kManyOutputs ? kLdsBudgetManyOutputs : kLdsBudget;
  int rb = 32;
  while (rb > 1 && (rb / 2 >= a.R || lds_floats(a, rb) * 4 > budget)) rb /= 2;
  return rb;
}

}  // namespace

bool fwd_general_supported(const FwdArgs& a) {
  return lds_floats(a, 1) * 4 <= kLdsBudget && a.N <= 65535 &&
         (geometry_of(a).Ho + kTH - 1) / kTH <= 65535;
}

template <int RB>
hipError_t launch_rb(const FwdArgs& a, size_t smem, hipStream_t s) {
  const void* fn = reinterpret_cast<const void*>(fwd_general_kernel<RB>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (e != hipSuccess) return e;
  const Geometry g = geometry_of(a);
  const dim3 grid((g.Wo + kTW - 1) / kTW, (g.Ho + kTH - 1) / kTH, a.N);
  fwd_general_kernel<RB><<<grid, kThreads, smem, s>>>(a, g);
  return hipGetLastError();
}

hipError_t fwd_general_launch(const FwdArgs& a, hipStream_t s) {
  const int rb = pick_rank_block(a);
  const size_t smem = lds_floats(a, rb) * sizeof(float);
  switch (rb) {
    case 32: return launch_rb<32>(a, smem, s);
    case 16: return launch_rb<16>(a, smem, s);
    case 8: return launch_rb<8>(a, smem, s);
    case 4: return launch_rb<4>(a, smem, s);
    case 2: return launch_rb<2>(a, smem, s);
    default: return launch_rb<1>(a, smem, s);
  }
}

}  // namespace cp4
