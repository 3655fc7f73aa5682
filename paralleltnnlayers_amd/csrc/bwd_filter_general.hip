// General backward-filter path: factor gradients for any shape, VALU
// arithmetic, intermediates in a caller-provided workspace.
//
// With A = FC^T x, B = FH *v A, Cc = FW *h B (the forward chain) and
// G3 = FK^T dy, G2 = adj_h(G3), G1 = adj_v(G2) (the backward chain), all
// [N,R,H,W], the reference's 8-deep sums
// (Cuda_kernels/cp4Conv2dBackwardFilter.cu:64-257) reassociate to
//   dFK[t,r] = sum_{n,p} dy[n,t,p] Cc[n,r,p]    dFC[c,r] = sum_{n,p} x[n,c,p] G1[n,r,p]
//   dFW[j,r] = sum G3[h,w] B[h,w+j-P]           dFH[i,r] = sum G2[h,w] A[h+i-P,w]
// Reductions are two-stage (per-workgroup partials in the workspace, then a
// fixed-order sum), so results are bit-reproducible run to run.
#include "cp4_internal.h"

namespace cp4 {
namespace {

constexpr int kThreads = 256;
constexpr int kRB = 16;  // rank block held in registers

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// Sum over the workgroup; result valid in thread 0.  `red` holds one float per wave.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wv] = v;
  __syncthreads();
  float s = 0.f;
  if (threadIdx.x == 0)
    for (int i = 0; i < kThreads / 64; ++i) s += red[i];
  return s;
}

// Z[n,r,p] = sum_c F[c,r] src[n,c,p]
__global__ __launch_bounds__(kThreads) void contract_in_kernel(
    const float* __restrict__ src, const float* __restrict__ F,
    float* __restrict__ Z, int Cin, int R, int HW) {
  const int p = blockIdx.x * kThreads + threadIdx.x;
  const int n = blockIdx.y, r0 = blockIdx.z * kRB;
  if (p >= HW) return;
  float acc[kRB];
#pragma unroll
  for (int rr = 0; rr < kRB; ++rr) acc[rr] = 0.f;
  const float* sp = src + (size_t)n * Cin * HW + p;
  for (int c = 0; c < Cin; ++c) {
    const float v = sp[(size_t)c * HW];
    const float* f = F + (size_t)c * R + r0;
#pragma unroll
    for (int rr = 0; rr < kRB; ++rr) acc[rr] += v * (r0 + rr < R ? f[rr] : 0.f);
  }
#pragma unroll
  for (int rr = 0; rr < kRB; ++rr)
    if (r0 + rr < R) Z[((size_t)n * R + r0 + rr) * HW + p] = acc[rr];
}

// Depthwise 1-D taps on [planes = N*R] planes of H x W.
// axis 0: along H, axis 1: along W.  adj 0: src index +t-P; adj 1: -t+P.
__global__ __launch_bounds__(kThreads) void depthwise_kernel(
    const float* __restrict__ src, const float* __restrict__ F,
    float* __restrict__ dst, size_t total, int R, int H, int W, int taps, int P,
    int axis, int adj) {
  const size_t idx = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int w = idx % W;
  const int h = (idx / W) % H;
  const size_t plane = idx / ((size_t)W * H);
  const int r = plane % R;
  const float* sp = src + plane * (size_t)H * W;
  float s = 0.f;
  for (int t = 0; t < taps; ++t) {
    const int o = adj ? P - t : t - P;
    const int hh = axis == 0 ? h + o : h, ww = axis == 1 ? w + o : w;
    if (hh >= 0 && hh < H && ww >= 0 && ww < W) s += F[t * R + r] * sp[hh * W + ww];
  }
  dst[idx] = s;
}

// partial[s][d][r] = sum_{n in split s, p} act[n,d,p] Z[n,r,p]
__global__ __launch_bounds__(kThreads) void grad_channel_kernel(
    const float* __restrict__ act, const float* __restrict__ Z,
    float* __restrict__ partial, int N, int D, int R, int HW, int S) {
  __shared__ float red[kThreads / 64];
  const int d = blockIdx.x, s = blockIdx.y;
  const int n0 = (int)((long)N * s / S), n1 = (int)((long)N * (s + 1) / S);
  for (int r0 = 0; r0 < R; r0 += kRB) {
    float acc[kRB];
#pragma unroll
    for (int rr = 0; rr < kRB; ++rr) acc[rr] = 0.f;
    for (int n = n0; n < n1; ++n) {
      const float* ap = act + ((size_t)n * D + d) * HW;
      const float* zp = Z + ((size_t)n * R + r0) * HW;
      for (int p = threadIdx.x; p < HW; p += kThreads) {
        const float v = ap[p];
#pragma unroll
        for (int rr = 0; rr < kRB; ++rr)
          if (r0 + rr < R) acc[rr] += v * zp[(size_t)rr * HW + p];
      }
    }
#pragma unroll
    for (int rr = 0; rr < kRB; ++rr) {
      const float t = block_sum(acc[rr], red);
      if (threadIdx.x == 0 && r0 + rr < R)
        partial[((size_t)s * D + d) * R + r0 + rr] = t;
    }
  }
}

// partial[s][t][r] = sum_{n in split s, h, w} P0[n,r,h,w] * P1[n,r,h+o,w] (axis 0)
// or P1[n,r,h,w+o] (axis 1), o = t - P.
__global__ __launch_bounds__(kThreads) void grad_tap_kernel(
    const float* __restrict__ P0, const float* __restrict__ P1,
    float* __restrict__ partial, int N, int R, int H, int W, int taps, int P,
    int axis, int S) {
  __shared__ float red[kThreads / 64];
  const int t = blockIdx.x, r = blockIdx.y, s = blockIdx.z;
  const int n0 = (int)((long)N * s / S), n1 = (int)((long)N * (s + 1) / S);
  const int o = t - P, HW = H * W;
  float acc = 0.f;
  for (int n = n0; n < n1; ++n) {
    const float* a = P0 + ((size_t)n * R + r) * HW;
    const float* b = P1 + ((size_t)n * R + r) * HW;
    for (int p = threadIdx.x; p < HW; p += kThreads) {
      const int h = p / W, w = p - h * W;
      const int hh = axis == 0 ? h + o : h, ww = axis == 1 ? w + o : w;
      if (hh >= 0 && hh < H && ww >= 0 && ww < W) acc += a[p] * b[hh * W + ww];
    }
  }
  const float tot = block_sum(acc, red);
  if (threadIdx.x == 0) partial[((size_t)s * taps + t) * R + r] = tot;
}

// out[i] = sum_s partial[s][i], fixed order.
__global__ __launch_bounds__(kThreads) void reduce_partials_kernel(
    const float* __restrict__ partial, float* __restrict__ out, int count, int S) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= count) return;
  float s = 0.f;
  for (int k = 0; k < S; ++k) s += partial[(size_t)k * count + i];
  out[i] = s;
}

// Dense gradient dK[t,c,y,x] (+)= sum_{n,h,w} dy[n,t,h,w] x[n,c,h+y-P,w+x-P]
// (Cuda_kernels/cp4Conv2dBackwardFilter.cu:47-56); one workgroup per (c,t).
__global__ __launch_bounds__(kThreads) void dense_filter_grad_kernel(
    const float* __restrict__ x, const float* __restrict__ dy,
    float* __restrict__ dK, int N, int C, int T, int H, int W, int P, int Y,
    int X, int accumulate) {
  __shared__ float red[kThreads / 64];
  const int c = blockIdx.x, t = blockIdx.y, HW = H * W;
  for (int fy = 0; fy < Y; ++fy)
    for (int fx = 0; fx < X; ++fx) {
      float acc = 0.f;
      for (int n = 0; n < N; ++n) {
        const float* xp = x + ((size_t)n * C + c) * HW;
        const float* gp = dy + ((size_t)n * T + t) * HW;
        for (int p = threadIdx.x; p < HW; p += kThreads) {
          const int h = p / W, w = p - h * W;
          const int hh = h + fy - P, ww = w + fx - P;
          if (hh >= 0 && hh < H && ww >= 0 && ww < W) acc += gp[p] * xp[hh * W + ww];
        }
      }
      const float tot = block_sum(acc, red);
      if (threadIdx.x == 0) {
        float* o = dK + (((size_t)t * C + c) * Y + fy) * X + fx;
        *o = accumulate ? *o + tot : tot;
      }
    }
}

// The same for square filters up to 7x7: all FS x FS taps of a (c,t) pair in one sweep over
// the pixels (the kernel above sweeps them once per tap), dy read once per pixel, the
// FS x FS neighbours of x mostly out of cache (N32 C16 K16 56x56 3x3: 1450 -> 200 us).
template <int FS>
__global__ __launch_bounds__(kThreads) void dense_filter_grad_taps_kernel(
    const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ dK, int N,
    int C, int T, int H, int W, int P, unsigned wmagic, int accumulate) {
  __shared__ float red[kThreads / 64];
  const int c = blockIdx.x, t = blockIdx.y, HW = H * W;
  float acc[FS][FS];
#pragma unroll
  for (int i = 0; i < FS; ++i)
#pragma unroll
    for (int j = 0; j < FS; ++j) acc[i][j] = 0.f;
  for (int n = 0; n < N; ++n) {
    const float* xp = x + ((size_t)n * C + c) * HW;
    const float* gp = dy + ((size_t)n * T + t) * HW;
    for (int p = threadIdx.x; p < HW; p += kThreads) {
      const int h = (int)__umulhi((unsigned)p, wmagic), w = p - h * W;
      const float g = gp[p];
#pragma unroll
      for (int i = 0; i < FS; ++i) {
        const int hh = h + i - P;
        const bool rin = hh >= 0 && hh < H;
        const float* row = xp + (rin ? hh : 0) * W;
#pragma unroll
        for (int j = 0; j < FS; ++j) {
          const int ww = w + j - P;
          const bool in = rin && ww >= 0 && ww < W;
          const float v = row[in ? ww : 0];
          acc[i][j] += in ? g * v : 0.f;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < FS; ++i)
#pragma unroll
    for (int j = 0; j < FS; ++j) {
      const float tot = block_sum(acc[i][j], red);
      if (threadIdx.x == 0) {
        float* o = dK + (((size_t)t * C + c) * FS + i) * FS + j;
        *o = accumulate ? *o + tot : tot;
      }
    }
}

int channel_splits(int N) { return N < 8 ? N : 8; }

}  // namespace

size_t bwd_filter_workspace_bytes(const cp4_shape& s) {
  const size_t plane = (size_t)s.N * s.Rank * s.H * s.W;
  const size_t S = channel_splits(s.N);
  const size_t partial = S * (size_t)s.Rank * ((size_t)s.T + s.C + s.Y + s.X);
  return (6 * plane + partial) * sizeof(float);
}

hipError_t bwd_filter_launch(const BwdFilterArgs& a, hipStream_t st) {
  const int HW = a.H * a.W, R = a.R, N = a.N;
  const size_t plane = (size_t)N * R * HW;
  float* ws = static_cast<float*>(a.workspace);
  float *A = ws, *B = ws + plane, *Cc = ws + 2 * plane, *G3 = ws + 3 * plane,
        *G2 = ws + 4 * plane, *G1 = ws + 5 * plane, *part = ws + 6 * plane;
  const int S = channel_splits(N);

  const dim3 cgrid((HW + kThreads - 1) / kThreads, N, (R + kRB - 1) / kRB);
  contract_in_kernel<<<cgrid, kThreads, 0, st>>>(a.x, a.FC, A, a.C, R, HW);
  contract_in_kernel<<<cgrid, kThreads, 0, st>>>(a.dy, a.FK, G3, a.T, R, HW);
  const unsigned dgrid = (unsigned)((plane + kThreads - 1) / kThreads);
  depthwise_kernel<<<dgrid, kThreads, 0, st>>>(A, a.FH, B, plane, R, a.H, a.W, a.Y, a.pad, 0, 0);
  depthwise_kernel<<<dgrid, kThreads, 0, st>>>(B, a.FW, Cc, plane, R, a.H, a.W, a.X, a.pad, 1, 0);
  depthwise_kernel<<<dgrid, kThreads, 0, st>>>(G3, a.FW, G2, plane, R, a.H, a.W, a.X, a.pad, 1, 1);
  depthwise_kernel<<<dgrid, kThreads, 0, st>>>(G2, a.FH, G1, plane, R, a.H, a.W, a.Y, a.pad, 0, 1);

  float* pK = part;
  float* pC = pK + (size_t)S * a.T * R;
  float* pH = pC + (size_t)S * a.C * R;
  float* pW = pH + (size_t)S * a.Y * R;
  grad_channel_kernel<<<dim3(a.T, S), kThreads, 0, st>>>(a.dy, Cc, pK, N, a.T, R, HW, S);
  grad_channel_kernel<<<dim3(a.C, S), kThreads, 0, st>>>(a.x, G1, pC, N, a.C, R, HW, S);
  grad_tap_kernel<<<dim3(a.Y, R, S), kThreads, 0, st>>>(G2, A, pH, N, R, a.H, a.W, a.Y, a.pad, 0, S);
  grad_tap_kernel<<<dim3(a.X, R, S), kThreads, 0, st>>>(G3, B, pW, N, R, a.H, a.W, a.X, a.pad, 1, S);
  auto reduce = [&](const float* p, float* out, int count) {
    reduce_partials_kernel<<<(count + kThreads - 1) / kThreads, kThreads, 0, st>>>(p, out, count, S);
  };
  reduce(pK, a.dFK, a.T * R);
  reduce(pC, a.dFC, a.C * R);
  reduce(pH, a.dFH, a.Y * R);
  reduce(pW, a.dFW, a.X * R);
  return hipGetLastError();
}

hipError_t bwd_filter_full_launch(const cp4_shape& s, const float* x,
                                  const float* dy, float* dK, int accumulate,
                                  hipStream_t st) {
  const unsigned wmagic = (unsigned)((0x100000000ull + s.W - 1) / s.W);   // ceil(2^32 / W)
  const dim3 grid(s.C, s.T);
  const bool taps = s.Y == s.X && (size_t)s.H * s.W < (1u << 24);   // (exact p / W by multiplication)
  if (taps && s.Y == 1)
    dense_filter_grad_taps_kernel<1><<<grid, kThreads, 0, st>>>(x, dy, dK, s.N, s.C, s.T, s.H, s.W,
                                                                 s.pad, wmagic, accumulate);
  else if (taps && s.Y == 3)
    dense_filter_grad_taps_kernel<3><<<grid, kThreads, 0, st>>>(x, dy, dK, s.N, s.C, s.T, s.H, s.W,
                                                                 s.pad, wmagic, accumulate);
  else if (taps && s.Y == 5)
    dense_filter_grad_taps_kernel<5><<<grid, kThreads, 0, st>>>(x, dy, dK, s.N, s.C, s.T, s.H, s.W,
                                                                 s.pad, wmagic, accumulate);
  else if (taps && s.Y == 7)
    dense_filter_grad_taps_kernel<7><<<grid, kThreads, 0, st>>>(x, dy, dK, s.N, s.C, s.T, s.H, s.W,
                                                                 s.pad, wmagic, accumulate);
  else
    dense_filter_grad_kernel<<<grid, kThreads, 0, st>>>(x, dy, dK, s.N, s.C, s.T, s.H, s.W, s.pad,
                                                        s.Y, s.X, accumulate);
  return hipGetLastError();
}

}  // namespace cp4
