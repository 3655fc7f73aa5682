// Test / bench utility kernels: filter recomposition, the reference's
// relative-error counter, a counter-based uniform generator and a streaming
// copy used for bandwidth and hardware-counter calibration.
#include "cp4_internal.h"

namespace cp4 {
namespace {

// K[t,c,y,x] = sum_r FK[t,r] FC[c,r] FH[y,r] FW[x,r]  (Cuda_kernels/Utils.cu:55-62)
__global__ __launch_bounds__(256) void recompose_kernel(
    const float* __restrict__ FK, const float* __restrict__ FC,
    const float* __restrict__ FH, const float* __restrict__ FW,
    float* __restrict__ K, int T, int C, int Y, int X, int R) {
  const size_t total = (size_t)T * C * Y * X;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (size_t)gridDim.x * 256) {
    const int x = i % X, y = (i / X) % Y, c = (i / ((size_t)X * Y)) % C;
    const int t = i / ((size_t)X * Y * C);
    float acc = 0.f;
    for (int r = 0; r < R; ++r)
      acc += FK[t * R + r] * FC[c * R + r] * FH[y * R + r] * FW[x * R + r];
    K[i] = acc;
  }
}

// Symmetric relative error, absolute if either value is zero
// (Cuda_kernels/Utils.cu:143-156); one integer atomic per workgroup.
__global__ __launch_bounds__(256) void count_exceeding_kernel(
    const float* __restrict__ A, const float* __restrict__ B, size_t n,
    float tol, unsigned long long* count) {
  unsigned bad = 0;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (size_t)gridDim.x * 256) {
    const float a = A[i], b = B[i], d = fabsf(a - b);
    const float err = (a == 0.f || b == 0.f) ? d : fmaxf(d / fabsf(a), d / fabsf(b));
    // NaN must count as a mismatch
    bad += !(err <= tol);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) bad += __shfl_down(bad, off, 64);
  if ((threadIdx.x & 63) == 0 && bad) atomicAdd(count, (unsigned long long)bad);
}

__device__ __forceinline__ unsigned long long splitmix64(unsigned long long z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// dst[i] in (0,1]: 24 random bits of hash(seed, i), like cuRAND's uniform
// range used by random_fill (Cuda_kernels/Utils.cu:22-33).
__global__ __launch_bounds__(256) void random_uniform_kernel(
    float* __restrict__ dst, size_t n, unsigned long long seed) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (size_t)gridDim.x * 256) {
    const unsigned long long h = splitmix64(splitmix64(seed) ^ i);
    dst[i] = ((float)(unsigned)(h >> 40) + 1.0f) * (1.0f / 16777216.0f);
  }
}

__global__ __launch_bounds__(256) void copy_f32x4_kernel(
    float4* __restrict__ dst, const float4* __restrict__ src, size_t n4) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4;
       i += (size_t)gridDim.x * 256)
    dst[i] = src[i];
}
// dst[g][r][e] = r < rows ? src[g][r][e] : 0 for r < rows_padded: matrices or image
// stacks with zero rows (channels) appended.  V = float4 when rows are whole quads.
template <class V>
__global__ __launch_bounds__(256) void pad_rows_kernel(V* __restrict__ dst,
                                                       const V* __restrict__ src, size_t groups,
                                                       size_t rows, size_t rows_padded,
                                                       size_t row_elems) {
  const size_t total = groups * rows_padded * row_elems;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (size_t)gridDim.x * 256) {
    const size_t e = i % row_elems, gr = i / row_elems;
    const size_t r = gr % rows_padded, g = gr / rows_padded;
    V v{};
    if (r < rows) v = src[(g * rows + r) * row_elems + e];
    dst[i] = v;
  }
}
__global__ __launch_bounds__(256) void add_f32_kernel(float* __restrict__ dst,
                                                      const float* __restrict__ src, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    dst[i] += src[i];
}
__global__ __launch_bounds__(256) void copy_f32_kernel(
    float* __restrict__ dst, const float* __restrict__ src, size_t lo, size_t n) {
  const size_t i = lo + (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void zero_f32_kernel(float* __restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (size_t)gridDim.x * 256)
    dst[i] = 0.f;
}

// dst[plane][ot + sh*h][ol + sw*w] = src[plane][h][w], every other cell of dst zero:
// a plane set into a larger canvas, its pixels spread sh x sw apart (zero
// insertion).  One pass that writes every cell of dst.
__global__ __launch_bounds__(256) void embed_kernel(const float* __restrict__ src,
                                                    float* __restrict__ dst, size_t planes, int h,
                                                    int w, int Hc, int Wc, int ot, int ol, int sh,
                                                    int sw) {
  const size_t total = planes * Hc * Wc;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (size_t)gridDim.x * 256) {
    const int v = (int)(i % Wc), u = (int)((i / Wc) % Hc);
    const size_t p = i / ((size_t)Wc * Hc);
    const int du = u - ot, dv = v - ol;
    float val = 0.f;
    if (du >= 0 && dv >= 0 && du % sh == 0 && dv % sw == 0 && du / sh < h && dv / sw < w)
      val = src[(p * h + du / sh) * w + dv / sw];
    dst[i] = val;
  }
}

// Reshaped-CP op: its dense filter from K0 [S0,T0,R], K1 [S1,T1,R], KC [Y,X,R]
// (test/test_conv2d_rcp.py:38-39): K[(x,y),(a,b),i,j] = sum_r K0[a,x,r] K1[b,y,r] KC[i,j,r].
// transposed == 0: out[T][C][Y][X]; != 0: the filter of the input-gradient pass,
// out[C][T][Y][X] with the taps reversed.
__global__ __launch_bounds__(256) void rcp_recompose_kernel(
    const float* __restrict__ K0, const float* __restrict__ K1, const float* __restrict__ KC,
    float* __restrict__ out, int S0, int S1, int T0, int T1, int Y, int X, int R, int transposed) {
  const int C = S0 * S1, T = T0 * T1;
  const size_t total = (size_t)T * C * Y * X;
  for (size_t q = (size_t)blockIdx.x * 256 + threadIdx.x; q < total; q += (size_t)gridDim.x * 256) {
    const int j = (int)(q % X), i = (int)((q / X) % Y);
    const int inner = (int)((q / ((size_t)X * Y)) % (transposed ? T : C));
    const int outer = (int)(q / ((size_t)X * Y * (transposed ? T : C)));
    const int t = transposed ? inner : outer, c = transposed ? outer : inner;
    const int ti = transposed ? Y - 1 - i : i, tj = transposed ? X - 1 - j : j;
    const int a = c / S1, b = c % S1, x = t / T1, y = t % T1;
    const float *p0 = K0 + (size_t)(a * T0 + x) * R, *p1 = K1 + (size_t)(b * T1 + y) * R,
                *p2 = KC + (size_t)(ti * X + tj) * R;
    float s = 0.f;
    for (int r = 0; r < R; ++r) s += p0[r] * p1[r] * p2[r];
    out[q] = s;
  }
}

// Chain rule from the dense filter gradient dK [T][C][Y][X] to the three factors:
// element e of [dK0 | dK1 | dKC] sums dK times the other two factors, fixed order.
__global__ __launch_bounds__(256) void rcp_fold_kernel(
    const float* __restrict__ dK, const float* __restrict__ K0, const float* __restrict__ K1,
    const float* __restrict__ KC, float* __restrict__ dK0, float* __restrict__ dK1,
    float* __restrict__ dKC, int S0, int S1, int T0, int T1, int Y, int X, int R) {
  const int C = S0 * S1;
  const int n0 = S0 * T0 * R, n1 = S1 * T1 * R, n2 = Y * X * R;
  for (int e = blockIdx.x * 256 + threadIdx.x; e < n0 + n1 + n2; e += gridDim.x * 256) {
    float s = 0.f;
    if (e < n0) {
      const int r = e % R, x = (e / R) % T0, a = e / (R * T0);
      for (int b = 0; b < S1; ++b)
        for (int y = 0; y < T1; ++y) {
          const float f1 = K1[(size_t)(b * T1 + y) * R + r];
          const float* g = dK + ((size_t)(x * T1 + y) * C + a * S1 + b) * Y * X;
          float u = 0.f;
          for (int ij = 0; ij < Y * X; ++ij) u += g[ij] * KC[(size_t)ij * R + r];
          s += f1 * u;
        }
      dK0[e] = s;
    } else if (e < n0 + n1) {
      const int q = e - n0, r = q % R, y = (q / R) % T1, b = q / (R * T1);
      for (int a = 0; a < S0; ++a)
        for (int x = 0; x < T0; ++x) {
          const float f0 = K0[(size_t)(a * T0 + x) * R + r];
          const float* g = dK + ((size_t)(x * T1 + y) * C + a * S1 + b) * Y * X;
          float u = 0.f;
          for (int ij = 0; ij < Y * X; ++ij) u += g[ij] * KC[(size_t)ij * R + r];
          s += f0 * u;
        }
      dK1[q] = s;
    } else {
      const int q = e - n0 - n1, r = q % R, ij = q / R;
      for (int a = 0; a < S0; ++a)
        for (int x = 0; x < T0; ++x) {
          const float f0 = K0[(size_t)(a * T0 + x) * R + r];
          float u = 0.f;
          for (int b = 0; b < S1; ++b)
            for (int y = 0; y < T1; ++y)
              u += dK[((size_t)(x * T1 + y) * C + a * S1 + b) * Y * X + ij] *
                   K1[(size_t)(b * T1 + y) * R + r];
          s += f0 * u;
        }
      dKC[q] = s;
    }
  }
}

// dst[row*ld_dst + c] = src[row*ld_src + c] for c < cols: a column block of a
// row-major matrix copied to or from a compact one.
__global__ __launch_bounds__(256) void copy_columns_kernel(const float* __restrict__ src,
                                                           int ld_src, float* __restrict__ dst,
                                                           int ld_dst, int rows, int cols) {
  const int total = rows * cols;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    const int row = i / cols, c = i - row * cols;
    dst[(size_t)row * ld_dst + c] = src[(size_t)row * ld_src + c];
  }
}

// one workgroup per (image, channel) plane segment: the bias is a scalar
__global__ __launch_bounds__(256) void bias_act_kernel(float* __restrict__ y,
                                                       const float* __restrict__ bias, int act,
                                                       size_t planes, size_t K, size_t HW) {
  for (size_t plane = blockIdx.x; plane < planes; plane += gridDim.x) {   // n * K + k
    const float b = bias ? bias[plane % K] : 0.f;
    float* row = y + plane * HW;
    for (size_t i = (size_t)blockIdx.y * 256 + threadIdx.x; i < HW;
         i += (size_t)gridDim.y * 256) {
      float v = row[i] + b;
      if (act) v = v < 0.f ? 0.f : v;
      row[i] = v;
    }
  }
}

// 3-factor CP (pointwise K0 [C,R], depthwise K1 [Y,X,R], pointwise K2 [R,T];
// Kernels/cp_fused_nchw.cc:20-24) written as a CP4 of rank Y*R: rank q = i*R + r
// stands for row i of the depthwise filter of rank r,
//   FC'[c,q] = K0[c,r]   FH'[y,q] = (y == i)   FW'[x,q] = K1[i,x,r]   FK'[t,q] = K2[r,t].
// The unit column taps only multiply by one and add zeros, so the CP4 kernels
// compute sum_r K2[r,t] sum_{i,x} K1[i,x,r] sum_c K0[c,r] x[...] with no extra rounding.
__global__ __launch_bounds__(256) void cp3_expand_kernel(
    const float* __restrict__ K0, const float* __restrict__ K1, const float* __restrict__ K2,
    float* __restrict__ FK, float* __restrict__ FC, float* __restrict__ FH,
    float* __restrict__ FW, int T, int C, int Y, int X, int R) {
  const size_t Q = (size_t)Y * R, total = (size_t)(T + C + Y + X) * Q;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * 256) {
    const size_t q = idx % Q;
    int row = (int)(idx / Q);
    const int i = (int)(q / R), r = (int)(q % R);
    if (row < T) {
      FK[(size_t)row * Q + q] = K2[(size_t)r * T + row];
    } else if ((row -= T) < C) {
      FC[(size_t)row * Q + q] = K0[(size_t)row * R + r];
    } else if ((row -= C) < Y) {
      FH[(size_t)row * Q + q] = row == i ? 1.f : 0.f;
    } else {
      row -= Y;
      FW[(size_t)row * Q + q] = K1[((size_t)i * X + row) * R + r];
    }
  }
}

// Gradients of the three CP factors from those of the expanded CP4 factors:
// K0[c,r] and K2[r,t] appear in Y expanded columns each (summed in row order),
// K1[i,x,r] in exactly one.
__global__ __launch_bounds__(256) void cp3_fold_kernel(
    const float* __restrict__ dFK, const float* __restrict__ dFC, const float* __restrict__ dFW,
    float* __restrict__ dK0, float* __restrict__ dK1, float* __restrict__ dK2,
    int T, int C, int Y, int X, int R) {
  const size_t Q = (size_t)Y * R;
  const size_t n0 = (size_t)C * R, n1 = (size_t)Y * X * R, n2 = (size_t)R * T;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < n0 + n1 + n2;
       idx += (size_t)gridDim.x * 256) {
    if (idx < n0) {
      const size_t c = idx / R, r = idx % R;
      float acc = 0.f;
      for (int i = 0; i < Y; ++i) acc += dFC[c * Q + (size_t)i * R + r];
      dK0[idx] = acc;
    } else if (idx < n0 + n1) {
      const size_t j = idx - n0, r = j % R, x = (j / R) % X, i = j / ((size_t)R * X);
      dK1[j] = dFW[x * Q + i * R + r];
    } else {
      const size_t j = idx - n0 - n1, t = j % T, r = j / T;
      float acc = 0.f;
      for (int i = 0; i < Y; ++i) acc += dFK[t * Q + (size_t)i * R + r];
      dK2[j] = acc;
    }
  }
}

// dst[c, r] = src[r, c] (the [R,T] pointwise factor of the 3-factor CP op as a [T,R] one)
__global__ __launch_bounds__(256) void transpose_f32_kernel(const float* __restrict__ src,
                                                            float* __restrict__ dst, int rows,
                                                            int cols) {
  const size_t total = (size_t)rows * cols;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * 256)
    dst[idx] = src[(idx % rows) * cols + idx / rows];
}

unsigned grid_for(size_t n, unsigned cap) {
  const size_t g = (n + 255) / 256;
  return (unsigned)(g < 1 ? 1 : g > cap ? cap : g);
}

}  // namespace

hipError_t recompose_launch(const cp4_shape& s, const float* FK, const float* FC,
                            const float* FH, const float* FW, float* K,
                            hipStream_t st) {
  const size_t total = (size_t)s.T * s.C * s.Y * s.X;
  recompose_kernel<<<grid_for(total, 65536), 256, 0, st>>>(FK, FC, FH, FW, K, s.T, s.C, s.Y, s.X, s.Rank);
  return hipGetLastError();
}

hipError_t count_exceeding_launch(const float* A, const float* B, size_t n,
                                  float tol, unsigned long long* d_count,
                                  hipStream_t st) {
  count_exceeding_kernel<<<grid_for(n, 4096), 256, 0, st>>>(A, B, n, tol, d_count);
  return hipGetLastError();
}

hipError_t random_uniform_launch(float* dst, size_t n, unsigned long long seed,
                                 hipStream_t st) {
  random_uniform_kernel<<<grid_for(n, 65536), 256, 0, st>>>(dst, n, seed);
  return hipGetLastError();
}

hipError_t bias_act_launch(float* y, const float* bias, int act, size_t N, size_t K, size_t HW,
                           hipStream_t st) {
  if (N * K == 0 || HW == 0 || (!bias && !act)) return hipSuccess;
  const unsigned segs = (unsigned)((HW + 4095) / 4096 > 64 ? 64 : (HW + 4095) / 4096);
  const size_t planes = N * K;
  const unsigned gx = (unsigned)(planes > (1u << 20) ? (1u << 20) : planes);
  bias_act_kernel<<<dim3(gx, segs), 256, 0, st>>>(y, bias, act, planes, K, HW);
  return hipGetLastError();
}

hipError_t zero_f32_launch(float* dst, size_t n, hipStream_t st) {
  if (n == 0) return hipSuccess;
  zero_f32_kernel<<<grid_for(n, 2048), 256, 0, st>>>(dst, n);
  return hipGetLastError();
}

hipError_t rcp_recompose_launch(const float* K0, const float* K1, const float* KC, float* out,
                                int S0, int S1, int T0, int T1, int Y, int X, int R,
                                int transposed, hipStream_t st) {
  const size_t total = (size_t)S0 * S1 * T0 * T1 * Y * X;
  rcp_recompose_kernel<<<grid_for(total, 4096), 256, 0, st>>>(K0, K1, KC, out, S0, S1, T0, T1, Y, X,
                                                             R, transposed);
  return hipGetLastError();
}

hipError_t rcp_fold_launch(const float* dK, const float* K0, const float* K1, const float* KC,
                           float* dK0, float* dK1, float* dKC, int S0, int S1, int T0, int T1,
                           int Y, int X, int R, hipStream_t st) {
  const size_t total = (size_t)R * (S0 * T0 + S1 * T1 + Y * X);
  rcp_fold_kernel<<<grid_for(total, 4096), 256, 0, st>>>(dK, K0, K1, KC, dK0, dK1, dKC, S0, S1, T0,
                                                        T1, Y, X, R);
  return hipGetLastError();
}

hipError_t copy_columns_launch(const float* src, int ld_src, float* dst, int ld_dst, int rows,
                               int cols, hipStream_t st) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  copy_columns_kernel<<<grid_for((size_t)rows * cols, 1024), 256, 0, st>>>(src, ld_src, dst, ld_dst,
                                                                          rows, cols);
  return hipGetLastError();
}

hipError_t embed_launch(const float* src, float* dst, size_t planes, int h, int w, int Hc, int Wc,
                        int ot, int ol, int sh, int sw, hipStream_t st) {
  const size_t total = planes * Hc * Wc;
  if (total == 0) return hipSuccess;
  embed_kernel<<<grid_for(total, 8192), 256, 0, st>>>(src, dst, planes, h, w, Hc, Wc, ot, ol, sh, sw);
  return hipGetLastError();
}

hipError_t cp3_expand_launch(const cp4_shape& s, const float* K0, const float* K1,
                             const float* K2, float* FK, float* FC, float* FH, float* FW,
                             hipStream_t st) {
  const size_t total = (size_t)(s.T + s.C + s.Y + s.X) * s.Y * s.Rank;
  cp3_expand_kernel<<<grid_for(total, 4096), 256, 0, st>>>(K0, K1, K2, FK, FC, FH, FW, s.T, s.C,
                                                          s.Y, s.X, s.Rank);
  return hipGetLastError();
}

hipError_t cp3_fold_launch(const cp4_shape& s, const float* dFK, const float* dFC,
                           const float* dFW, float* dK0, float* dK1, float* dK2,
                           hipStream_t st) {
  const size_t total = (size_t)s.Rank * (s.C + s.T + (size_t)s.Y * s.X);
  cp3_fold_kernel<<<grid_for(total, 4096), 256, 0, st>>>(dFK, dFC, dFW, dK0, dK1, dK2, s.T, s.C,
                                                        s.Y, s.X, s.Rank);
  return hipGetLastError();
}

hipError_t transpose_f32_launch(const float* src, float* dst, int rows, int cols,
                                hipStream_t st) {
  transpose_f32_kernel<<<grid_for((size_t)rows * cols, 4096), 256, 0, st>>>(src, dst, rows, cols);
  return hipGetLastError();
}

hipError_t pad_rows_launch(const float* src, float* dst, size_t groups, size_t rows,
                           size_t rows_padded, size_t row_elems, hipStream_t st) {
  const size_t total = groups * rows_padded * row_elems;
  if (total == 0) return hipSuccess;
  if ((row_elems & 3) == 0 && (((uintptr_t)dst | (uintptr_t)src) & 15) == 0)
    pad_rows_kernel<float4><<<grid_for(total / 4, 2048), 256, 0, st>>>(
        reinterpret_cast<float4*>(dst), reinterpret_cast<const float4*>(src), groups, rows,
        rows_padded, row_elems / 4);
  else
    pad_rows_kernel<float><<<grid_for(total, 2048), 256, 0, st>>>(dst, src, groups, rows,
                                                                  rows_padded, row_elems);
  return hipGetLastError();
}

hipError_t add_f32_launch(float* dst, const float* src, size_t n, hipStream_t st) {
  if (n == 0) return hipSuccess;
  add_f32_kernel<<<grid_for(n, 2048), 256, 0, st>>>(dst, src, n);
  return hipGetLastError();
}

hipError_t copy_f32_launch(float* dst, const float* src, size_t n, hipStream_t st) {
  const bool aligned = (((uintptr_t)dst | (uintptr_t)src) & 15) == 0;
  const size_t n4 = aligned ? n / 4 : 0;
  if (n4) {
    // 256 CUs x 8 workgroups, grid-stride
    copy_f32x4_kernel<<<grid_for(n4, 2048), 256, 0, st>>>(
        reinterpret_cast<float4*>(dst), reinterpret_cast<const float4*>(src), n4);
  }
  const size_t rest = n - n4 * 4;
  if (rest)
    copy_f32_kernel<<<(unsigned)((rest + 255) / 256), 256, 0, st>>>(dst, src, n4 * 4, n);
  return hipGetLastError();
}

}  // namespace cp4
