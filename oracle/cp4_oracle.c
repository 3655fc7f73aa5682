/*
 * CPU oracle for the fused CP4-decomposed Conv2d (forward, backward-data,
 * backward-filter).  TEST INFRASTRUCTURE ONLY: this file is the checker that
 * the HIP kernels are compared against and the CPU baseline that the bench
 * reports beside the GPU number.  Nothing in the shipped library calls it.
 *
 * Two independent restatements live here:
 *
 *  (1) "direct" functions: literal loop nests over the defining formulas of
 *      the reference (slow, tiny shapes only):
 *        forward        Cuda_kernels/cp4Conv2dForward.cu:84-133
 *        backward-data  Cuda_kernels/cp4Conv2dBackwardData.cu:57-108
 *        filter grads   Cuda_kernels/cp4Conv2dBackwardFilter.cu:23-257
 *        recomposition  Cuda_kernels/Utils.cu:55-62
 *        comparator     Cuda_kernels/Utils.cu:143-156
 *        3-factor CP    test/layers.py:265-282 (forward only; its gradients are
 *                       checked against float64 autograd in the GPU tests)
 *        reshaped CP    test/test_conv2d_rcp.py:38-41 (forward only, likewise)
 *        strides etc.   test/layers.py:264-279 (section 1b: all three passes with a
 *                       stride, explicit padding and an output plane of its own)
 *
 *  (2) "unfused" functions: the factor-by-factor sequence
 *        1x1 conv by FC -> depthwise 1-D conv by FH -> depthwise 1-D conv by
 *        FW -> 1x1 conv by FK
 *      (the 4-factor form of test/layers.py:265-283 with the depthwise kernel
 *      FH (x) FW, i.e. test/test_conv2d_cp4.py:25), the transposed sequence
 *      with the reference's flipped taps for backward-data, and the factor
 *      gradients evaluated from the saved intermediates.  OpenMP over images;
 *      these are what the GPU results are compared with at full size and what
 *      the bench times as the CPU baseline.
 *
 * Factor order everywhere: FK[T,R] (out-channel, "FT" in the reference),
 * FC[C,R], FH[Y,R] ("FY"), FW[X,R] ("FX"); row-major; activations NCHW.
 * The output always has the input's H x W (the reference writes H x W
 * whatever pad is); taps that fall outside the image read zero.
 *
 * Pinning (see tests/test_oracle.py): (2) is checked against (1); (1) is
 * checked against torch's CPU dense conv2d / autograd on the recomposed
 * kernel, closed forms, the adjoint identity and the committed golden vectors.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct cp4o_shape {
  unsigned N, H, W, pad, T, C, Y, X, Rank; /* Cuda_kernels/Tensor.cuh:10-19 */
} cp4o_shape;

int cp4o_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------------ */
/* (1) direct restatements                                                   */
/* ------------------------------------------------------------------------ */

/* K[t,c,y,x] = sum_r FK[t,r] FC[c,r] FH[y,r] FW[x,r]   (Utils.cu:55-62) */
void cp4o_recompose(const cp4o_shape* s, const float* FK, const float* FC,
                    const float* FH, const float* FW, float* K) {
  const unsigned R = s->Rank;
  for (unsigned t = 0; t < s->T; ++t)
    for (unsigned c = 0; c < s->C; ++c)
      for (unsigned y = 0; y < s->Y; ++y)
        for (unsigned x = 0; x < s->X; ++x) {
          float acc = 0.0f;
          for (unsigned r = 0; r < R; ++r)
            acc += FK[t * R + r] * FC[c * R + r] * FH[y * R + r] * FW[x * R + r];
          K[((size_t)(t * s->C + c) * s->Y + y) * s->X + x] = acc;
        }
}

/* Zero-padded read of an NCHW plane. */
static inline double rd(const float* p, long h, long w, long H, long W) {
  return (h >= 0 && h < H && w >= 0 && w < W) ? (double)p[h * W + w] : 0.0;
}

/* Out[n,t,h,w] = sum_c sum_r FK[t,r] FC[c,r] sum_{y,x} FH[y,r] FW[x,r]
 *                In[n,c,h+y-pad,w+x-pad]      (cp4Conv2dForward.cu:84-133) */
void cp4o_forward_direct(const cp4o_shape* s, const float* In, const float* FK,
                         const float* FC, const float* FH, const float* FW,
                         float* Out) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X, R = s->Rank;
  for (long n = 0; n < N; ++n)
    for (long t = 0; t < T; ++t)
      for (long h = 0; h < H; ++h)
        for (long w = 0; w < W; ++w) {
          double acc = 0.0;
          for (long r = 0; r < R; ++r) {
            double cacc = 0.0;
            for (long c = 0; c < C; ++c) {
              const float* ip = In + (n * C + c) * H * W;
              double pix = 0.0;
              for (long y = 0; y < Y; ++y)
                for (long x = 0; x < X; ++x)
                  pix += rd(ip, h + y - P, w + x - P, H, W) *
                         (double)FH[y * R + r] * (double)FW[x * R + r];
              cacc += pix * (double)FC[c * R + r];
            }
            acc += cacc * (double)FK[t * R + r];
          }
          Out[((n * T + t) * H + h) * W + w] = (float)acc;
        }
}

/* 3-factor CP sibling op, as the reference's Python layer defines it
 * (test/layers.py:265-282: 1x1 conv by K0 [C,R], depthwise conv by K1 [Y,X,R],
 * 1x1 conv by K2 [R,T]; Kernels/cp_fused_nchw.cc:20-24 for the layouts), same
 * H x W output and zero reads outside the image as everywhere in this file:
 *   Out[n,t,h,w] = sum_r K2[r,t] sum_{y,x} K1[y,x,r] sum_c K0[c,r]
 *                  In[n,c,h+y-pad,w+x-pad]
 * Pinned in tests/test_oracle.py against torch's dense conv2d on the kernel
 * einsum('cr,ijr,rt->tcij') of test/test_conv2d_cp.py:20. */
void cp3o_forward_direct(const cp4o_shape* s, const float* In, const float* K0,
                         const float* K1, const float* K2, float* Out) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X, R = s->Rank;
  double* u0 = (double*)malloc(sizeof(double) * (size_t)(R * H * W));
  double* u1 = (double*)malloc(sizeof(double) * (size_t)(R * H * W));
  for (long n = 0; n < N; ++n) {
    for (long r = 0; r < R; ++r)
      for (long q = 0; q < H * W; ++q) {
        double acc = 0.0;
        for (long c = 0; c < C; ++c)
          acc += (double)In[(n * C + c) * H * W + q] * (double)K0[c * R + r];
        u0[r * H * W + q] = acc;
      }
    for (long r = 0; r < R; ++r)
      for (long h = 0; h < H; ++h)
        for (long w = 0; w < W; ++w) {
          double acc = 0.0;
          for (long y = 0; y < Y; ++y)
            for (long x = 0; x < X; ++x) {
              const long hh = h + y - P, ww = w + x - P;
              if (hh >= 0 && hh < H && ww >= 0 && ww < W)
                acc += u0[(r * H + hh) * W + ww] * (double)K1[(y * X + x) * R + r];
            }
          u1[(r * H + h) * W + w] = acc;
        }
    for (long t = 0; t < T; ++t)
      for (long q = 0; q < H * W; ++q) {
        double acc = 0.0;
        for (long r = 0; r < R; ++r) acc += u1[r * H * W + q] * (double)K2[r * T + t];
        Out[(n * T + t) * H * W + q] = (float)acc;
      }
  }
  free(u0);
  free(u1);
}

/* dx[n,c,h,w] = sum_r FC[c,r] sum_t FK[t,r] sum_{y,x} FH[Y-1-y,r] FW[X-1-x,r]
 *               dy[n,t,h+y-pad,w+x-pad]   (cp4Conv2dBackwardData.cu:57-108) */
void cp4o_backward_data_direct(const cp4o_shape* s, const float* dY,
                               const float* FK, const float* FC,
                               const float* FH, const float* FW, float* dX) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X, R = s->Rank;
  for (long n = 0; n < N; ++n)
    for (long c = 0; c < C; ++c)
      for (long h = 0; h < H; ++h)
        for (long w = 0; w < W; ++w) {
          double acc = 0.0;
          for (long r = 0; r < R; ++r) {
            double tacc = 0.0;
            for (long t = 0; t < T; ++t) {
              const float* ip = dY + (n * T + t) * H * W;
              double pix = 0.0;
              for (long y = 0; y < Y; ++y)
                for (long x = 0; x < X; ++x)
                  pix += rd(ip, h + y - P, w + x - P, H, W) *
                         (double)FH[(Y - 1 - y) * R + r] *
                         (double)FW[(X - 1 - x) * R + r];
              tacc += pix * (double)FK[t * R + r];
            }
            acc += tacc * (double)FC[c * R + r];
          }
          dX[((n * C + c) * H + h) * W + w] = (float)acc;
        }
}

/* dK[t,c,y,x] += sum_{n,h,w} dy[n,t,h,w] xpad[n,c,h+y,w+x]
 * (cp4Conv2dBackwardFilter.cu:23-59; xpad[h+y] == x[h+y-pad], zero outside) */
void cp4o_backward_filter_full_direct(const cp4o_shape* s, float* dK,
                                      const float* In, const float* dY) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X;
  for (long t = 0; t < T; ++t)
    for (long c = 0; c < C; ++c)
      for (long y = 0; y < Y; ++y)
        for (long x = 0; x < X; ++x) {
          double acc = 0.0;
          for (long n = 0; n < N; ++n) {
            const float* ip = In + (n * C + c) * H * W;
            const float* gp = dY + (n * T + t) * H * W;
            for (long h = 0; h < H; ++h)
              for (long w = 0; w < W; ++w)
                acc += (double)gp[h * W + w] * rd(ip, h + y - P, w + x - P, H, W);
          }
          dK[((t * C + c) * Y + y) * X + x] += (float)acc;
        }
}

/* The four factor gradients, literal 8-deep sums
 * (cp4Conv2dBackwardFilter.cu:64-107, 112-158, 163-208, 213-257).  `which`
 * selects the output: 0 dFK[t,r], 1 dFC[c,r], 2 dFH[y,r], 3 dFW[x,r].  All
 * four factors are passed; the one being differentiated is ignored.  The
 * output is accumulated into (+=) as in the reference. */
void cp4o_backward_filter_factor_direct(const cp4o_shape* s, int which,
                                        float* dF, const float* In,
                                        const float* dY, const float* FK,
                                        const float* FC, const float* FH,
                                        const float* FW) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X, R = s->Rank;
  const long D = which == 0 ? T : which == 1 ? C : which == 2 ? Y : X;
  for (long d = 0; d < D; ++d)
    for (long r = 0; r < R; ++r) {
      double acc = 0.0;
      for (long n = 0; n < N; ++n)
        for (long t = 0; t < T; ++t) {
          if (which == 0 && t != d) continue;
          for (long c = 0; c < C; ++c) {
            if (which == 1 && c != d) continue;
            const float* ip = In + (n * C + c) * H * W;
            const float* gp = dY + (n * T + t) * H * W;
            for (long y = 0; y < Y; ++y) {
              if (which == 2 && y != d) continue;
              for (long x = 0; x < X; ++x) {
                if (which == 3 && x != d) continue;
                double f = 1.0;
                if (which != 0) f *= (double)FK[t * R + r];
                if (which != 1) f *= (double)FC[c * R + r];
                if (which != 2) f *= (double)FH[y * R + r];
                if (which != 3) f *= (double)FW[x * R + r];
                double sum = 0.0;
                for (long h = 0; h < H; ++h)
                  for (long w = 0; w < W; ++w)
                    sum += (double)gp[h * W + w] *
                           rd(ip, h + y - P, w + x - P, H, W);
                acc += sum * f;
              }
            }
          }
        }
      dF[d * R + r] += (float)acc;
    }
}

/* ------------------------------------------------------------------------ */
/* (1b) layer geometry: stride and an output plane of its own                 */
/* ------------------------------------------------------------------------ */

/* The reference's kernels are stride 1 with an H x W output; its Python layer
 * passes strides and padding = "SAME" / "VALID" to the framework's convolutions
 * (test/layers.py:264-279).  With stride (sh, sw), pad_top / pad_left zero rows /
 * columns before the image and an out_h x out_w output plane the operator is
 *   Out[n,t,ho,wo] = sum_{c,r} FK[t,r] FC[c,r] sum_{y,x} FH[y,r] FW[x,r]
 *                    In[n,c, sh*ho + y - pad_top, sw*wo + x - pad_left]
 * (reads outside the image are zero), the forward formula of
 * cp4Conv2dForward.cu:84-133 with the anchor sh*ho, sw*wo in place of h, w.
 * s->pad is not used by the functions of this section.  Pinned in
 * tests/test_oracle.py against torch float64 conv2d(stride, padding) and its
 * autograd on the recomposed kernel (tests/golden/make_golden.py). */
typedef struct cp4o_geometry {
  unsigned stride_h, stride_w, pad_top, pad_left, out_h, out_w;
} cp4o_geometry;

void cp4o_forward_geom_direct(const cp4o_shape* s, const cp4o_geometry* g, const float* In,
                              const float* FK, const float* FC, const float* FH,
                              const float* FW, float* Out) {
  const long N = s->N, H = s->H, W = s->W, T = s->T, C = s->C, Y = s->Y, X = s->X, R = s->Rank;
  const long SH = g->stride_h, SW = g->stride_w, PT = g->pad_top, PL = g->pad_left,
             HO = g->out_h, WO = g->out_w;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (long n = 0; n < N; ++n)
    for (long t = 0; t < T; ++t)
      for (long ho = 0; ho < HO; ++ho)
        for (long wo = 0; wo < WO; ++wo) {
          double acc = 0.0;
          for (long r = 0; r < R; ++r) {
            double cacc = 0.0;
            for (long c = 0; c < C; ++c) {
              const float* ip = In + (n * C + c) * H * W;
              double pix = 0.0;
              for (long y = 0; y < Y; ++y)
                for (long x = 0; x < X; ++x)
                  pix += rd(ip, SH * ho + y - PT, SW * wo + x - PL, H, W) *
                         (double)FH[y * R + r] * (double)FW[x * R + r];
              cacc += pix * (double)FC[c * R + r];
            }
            acc += cacc * (double)FK[t * R + r];
          }
          Out[((n * T + t) * HO + ho) * WO + wo] = (float)acc;
        }
}

/* The adjoint of the map above in In: dX[n,c,h,w] = sum over every (t, ho, wo, y, x)
 * with sh*ho + y - pad_top = h and sw*wo + x - pad_left = w of
 * dY[n,t,ho,wo] K[t,c,y,x].  For stride 1, out = H x W and 2*pad = Y - 1 this is
 * cp4Conv2dBackwardData.cu:57-108. */
void cp4o_backward_data_geom_direct(const cp4o_shape* s, const cp4o_geometry* g,
                                    const float* dY, const float* FK, const float* FC,
                                    const float* FH, const float* FW, float* dX) {
  const long N = s->N, H = s->H, W = s->W, T = s->T, C = s->C, Y = s->Y, X = s->X, R = s->Rank;
  const long SH = g->stride_h, SW = g->stride_w, PT = g->pad_top, PL = g->pad_left,
             HO = g->out_h, WO = g->out_w;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (long n = 0; n < N; ++n)
    for (long c = 0; c < C; ++c)
      for (long h = 0; h < H; ++h)
        for (long w = 0; w < W; ++w) {
          double acc = 0.0;
          for (long r = 0; r < R; ++r) {
            double tacc = 0.0;
            for (long t = 0; t < T; ++t) {
              const float* gp = dY + (n * T + t) * HO * WO;
              double pix = 0.0;
              for (long y = 0; y < Y; ++y) {
                const long hn = h + PT - y;
                if (hn < 0 || hn % SH) continue;
                for (long x = 0; x < X; ++x) {
                  const long wn = w + PL - x;
                  if (wn < 0 || wn % SW) continue;
                  pix += rd(gp, hn / SH, wn / SW, HO, WO) * (double)FH[y * R + r] *
                         (double)FW[x * R + r];
                }
              }
              tacc += pix * (double)FK[t * R + r];
            }
            acc += tacc * (double)FC[c * R + r];
          }
          dX[((n * C + c) * H + h) * W + w] = (float)acc;
        }
}

/* The factor gradients of the map above, the 8-deep sums of
 * cp4Conv2dBackwardFilter.cu:64-257 with the strided anchor; `which` and the
 * += convention as in cp4o_backward_filter_factor_direct. */
void cp4o_backward_filter_geom_direct(const cp4o_shape* s, const cp4o_geometry* g, int which,
                                      float* dF, const float* In, const float* dY,
                                      const float* FK, const float* FC, const float* FH,
                                      const float* FW) {
  const long N = s->N, H = s->H, W = s->W, T = s->T, C = s->C, Y = s->Y, X = s->X, R = s->Rank;
  const long SH = g->stride_h, SW = g->stride_w, PT = g->pad_top, PL = g->pad_left,
             HO = g->out_h, WO = g->out_w;
  const long D = which == 0 ? T : which == 1 ? C : which == 2 ? Y : X;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (long d = 0; d < D; ++d)
    for (long r = 0; r < R; ++r) {
      double acc = 0.0;
      for (long n = 0; n < N; ++n)
        for (long t = 0; t < T; ++t) {
          if (which == 0 && t != d) continue;
          for (long c = 0; c < C; ++c) {
            if (which == 1 && c != d) continue;
            const float* ip = In + (n * C + c) * H * W;
            const float* gp = dY + (n * T + t) * HO * WO;
            for (long y = 0; y < Y; ++y) {
              if (which == 2 && y != d) continue;
              for (long x = 0; x < X; ++x) {
                if (which == 3 && x != d) continue;
                double f = 1.0;
                if (which != 0) f *= (double)FK[t * R + r];
                if (which != 1) f *= (double)FC[c * R + r];
                if (which != 2) f *= (double)FH[y * R + r];
                if (which != 3) f *= (double)FW[x * R + r];
                double sum = 0.0;
                for (long ho = 0; ho < HO; ++ho)
                  for (long wo = 0; wo < WO; ++wo)
                    sum += (double)gp[ho * WO + wo] *
                           rd(ip, SH * ho + y - PT, SW * wo + x - PL, H, W);
                acc += sum * f;
              }
            }
          }
        }
      dF[d * R + r] += (float)acc;
    }
}

/* The forward map above, factor by factor (1x1 by FC, strided depthwise 1-D by FH,
 * strided depthwise 1-D by FW, 1x1 by FK): what full-size results are compared
 * with.  Checked against cp4o_forward_geom_direct in tests/test_oracle.py. */
int cp4o_forward_geom_unfused(const cp4o_shape* s, const cp4o_geometry* g, const float* In,
                              const float* FK, const float* FC, const float* FH,
                              const float* FW, float* Out) {
  const long N = s->N, H = s->H, W = s->W, T = s->T, C = s->C, Y = s->Y, X = s->X, R = s->Rank;
  const long SH = g->stride_h, SW = g->stride_w, PT = g->pad_top, PL = g->pad_left,
             HO = g->out_h, WO = g->out_w, HW = H * W;
  int fail = 0;
#pragma omp parallel
  {
    float* a = (float*)malloc(sizeof(float) * (size_t)(R * HW));
    float* b = (float*)malloc(sizeof(float) * (size_t)(R * HO * W));
    float* cc = (float*)malloc(sizeof(float) * (size_t)(R * HO * WO));
    if (!a || !b || !cc) {
#pragma omp atomic write
      fail = 1;
    }
#pragma omp for schedule(dynamic)
    for (long n = 0; n < N; ++n) {
      if (!a || !b || !cc) continue;
      const float* xn = In + n * C * HW;
      for (long r = 0; r < R; ++r) {
        float* ar = a + r * HW;
        for (long p = 0; p < HW; ++p) ar[p] = 0.f;
        for (long c = 0; c < C; ++c) {
          const float f = FC[c * R + r];
          const float* xp = xn + c * HW;
          for (long p = 0; p < HW; ++p) ar[p] += f * xp[p];
        }
        float* br = b + r * HO * W;
        for (long ho = 0; ho < HO; ++ho)
          for (long w = 0; w < W; ++w) {
            float v = 0.f;
            for (long y = 0; y < Y; ++y) {
              const long h = SH * ho + y - PT;
              if (h >= 0 && h < H) v += FH[y * R + r] * ar[h * W + w];
            }
            br[ho * W + w] = v;
          }
        float* cr = cc + r * HO * WO;
        for (long ho = 0; ho < HO; ++ho)
          for (long wo = 0; wo < WO; ++wo) {
            float v = 0.f;
            for (long x = 0; x < X; ++x) {
              const long w = SW * wo + x - PL;
              if (w >= 0 && w < W) v += FW[x * R + r] * br[ho * W + w];
            }
            cr[ho * WO + wo] = v;
          }
      }
      for (long t = 0; t < T; ++t) {
        float* op = Out + (n * T + t) * HO * WO;
        for (long p = 0; p < HO * WO; ++p) op[p] = 0.f;
        for (long r = 0; r < R; ++r) {
          const float f = FK[t * R + r];
          const float* cr = cc + r * HO * WO;
          for (long p = 0; p < HO * WO; ++p) op[p] += f * cr[p];
        }
      }
    }
    free(a);
    free(b);
    free(cc);
  }
  return fail;
}

/* ------------------------------------------------------------------------ */
/* (1c) reshaped-CP sibling op                                               */
/* ------------------------------------------------------------------------ */

/* The reference's third fused op, Conv2dRcpFusedNchw (Kernels/rcp_fused_nchw.cc:6-12,
 * a generated kernel for the single shape 1 x (4,4) x 32 x 32, rank 11), as its test
 * defines it (test/test_conv2d_rcp.py:38-41): the input channels are the pairs (a, b)
 * of an S0 x S1 grid, the output channels the pairs (x, y) of a T0 x T1 grid, and the
 * dense filter is einsum('axr,byr,hwr->hwabxy') of K0 [S0,T0,R], K1 [S1,T1,R],
 * KC [Y,X,R], used in a "SAME" convolution:
 *   Out[n,(x,y),h,w] = sum_{a,b,i,j,r} K0[a,x,r] K1[b,y,r] KC[i,j,r]
 *                      In[n,(a,b),h+i-pad,w+j-pad]
 * with channel (a,b) = a*S1 + b and (x,y) = x*T1 + y (row-major reshapes).  s->C must
 * be S0*S1 and s->T = T0*T1.  Pinned in tests/test_oracle.py against torch's dense
 * conv2d on that einsum. */
void rcpo_forward_direct(const cp4o_shape* s, unsigned S0, unsigned S1, unsigned T0,
                         unsigned T1, const float* In, const float* K0, const float* K1,
                         const float* KC, float* Out) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, Y = s->Y, X = s->X, R = s->Rank;
  const long C = (long)S0 * S1, T = (long)T0 * T1;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (long n = 0; n < N; ++n)
    for (long t = 0; t < T; ++t) {
      const long x = t / T1, y = t % T1;
      for (long h = 0; h < H; ++h)
        for (long w = 0; w < W; ++w) {
          double acc = 0.0;
          for (long r = 0; r < R; ++r) {
            double cacc = 0.0;
            for (long c = 0; c < C; ++c) {
              const long a = c / S1, b = c % S1;
              const float* ip = In + (n * C + c) * H * W;
              double pix = 0.0;
              for (long i = 0; i < Y; ++i)
                for (long j = 0; j < X; ++j)
                  pix += rd(ip, h + i - P, w + j - P, H, W) * (double)KC[(i * X + j) * R + r];
              cacc += pix * (double)K0[(a * T0 + x) * R + r] * (double)K1[(b * T1 + y) * R + r];
            }
            acc += cacc;
          }
          Out[((n * T + t) * H + h) * W + w] = (float)acc;
        }
    }
}

/* Number of elements whose symmetric relative error exceeds tol; absolute
 * error when either value is zero (Utils.cu:143-156). */
long cp4o_count_exceeding(const float* A, const float* B, size_t n, float tol) {
  long bad = 0;
  for (size_t i = 0; i < n; ++i) {
    float a = A[i], b = B[i], d = fabsf(a - b);
    float err = (a == 0 || b == 0) ? d : fmaxf(d / fabsf(a), d / fabsf(b));
    if (err > tol) ++bad;
  }
  return bad;
}

/* ------------------------------------------------------------------------ */
/* (2) unfused factor-by-factor sequence                                     */
/* ------------------------------------------------------------------------ */

/* dst[r,p] = sum_c F[c,r] src[c,p]   (1x1 conv, channels Cin -> Cout=R cols) */
static void pointwise_in(const float* src, const float* F, float* dst, long Cin,
                         long R, long HW) {
  memset(dst, 0, sizeof(float) * (size_t)(R * HW));
  for (long c = 0; c < Cin; ++c) {
    const float* sp = src + c * HW;
    for (long r = 0; r < R; ++r) {
      const float f = F[c * R + r];
      float* dp = dst + r * HW;
      for (long p = 0; p < HW; ++p) dp[p] += f * sp[p];
    }
  }
}

/* dst[k,p] = sum_r F[k,r] src[r,p]   (1x1 conv, R -> Cout channels) */
static void pointwise_out(const float* src, const float* F, float* dst,
                          long Cout, long R, long HW) {
  for (long k = 0; k < Cout; ++k) {
    float* dp = dst + k * HW;
    memset(dp, 0, sizeof(float) * (size_t)HW);
    for (long r = 0; r < R; ++r) {
      const float f = F[k * R + r];
      const float* sp = src + r * HW;
      for (long p = 0; p < HW; ++p) dp[p] += f * sp[p];
    }
  }
}

/* Depthwise 1-D conv along H: dst[r,h,w] = sum_i F[tap(i),r] src[r,h+i-P,w].
 * flip selects tap(i) = Y-1-i (backward-data) instead of i. */
static void depthwise_v(const float* src, const float* F, float* dst, long R,
                        long H, long W, long Y, long P, int flip) {
  for (long r = 0; r < R; ++r)
    for (long h = 0; h < H; ++h) {
      float* dp = dst + (r * H + h) * W;
      memset(dp, 0, sizeof(float) * (size_t)W);
      for (long i = 0; i < Y; ++i) {
        const long hh = h + i - P;
        if (hh < 0 || hh >= H) continue;
        const float f = F[(flip ? Y - 1 - i : i) * R + r];
        const float* sp = src + (r * H + hh) * W;
        for (long w = 0; w < W; ++w) dp[w] += f * sp[w];
      }
    }
}

/* Depthwise 1-D conv along W: dst[r,h,w] = sum_j F[tap(j),r] src[r,h,w+j-P]. */
static void depthwise_h(const float* src, const float* F, float* dst, long R,
                        long H, long W, long X, long P, int flip) {
  for (long r = 0; r < R; ++r)
    for (long h = 0; h < H; ++h) {
      float* dp = dst + (r * H + h) * W;
      const float* sp = src + (r * H + h) * W;
      memset(dp, 0, sizeof(float) * (size_t)W);
      for (long j = 0; j < X; ++j) {
        const float f = F[(flip ? X - 1 - j : j) * R + r];
        const long lo = P - j > 0 ? P - j : 0;
        const long hi = W + P - j < W ? W + P - j : W;
        for (long w = lo; w < hi; ++w) dp[w] += f * sp[w + j - P];
      }
    }
}

int cp4o_forward_unfused(const cp4o_shape* s, const float* In, const float* FK,
                         const float* FC, const float* FH, const float* FW,
                         float* Out) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X, R = s->Rank, HW = H * W;
  int fail = 0;
#pragma omp parallel
  {
    float* a = (float*)malloc(sizeof(float) * (size_t)(R * HW));
    float* b = (float*)malloc(sizeof(float) * (size_t)(R * HW));
    if (!a || !b) {
#pragma omp atomic write
      fail = 1;
    }
#pragma omp for schedule(dynamic)
    for (long n = 0; n < N; ++n) {
      if (!a || !b) continue;
      pointwise_in(In + n * C * HW, FC, a, C, R, HW);
      depthwise_v(a, FH, b, R, H, W, Y, P, 0);
      depthwise_h(b, FW, a, R, H, W, X, P, 0);
      pointwise_out(a, FK, Out + n * T * HW, T, R, HW);
    }
    free(a);
    free(b);
  }
  return fail;
}

/* Transposed sequence with the reference's flipped taps:
 * 1x1 by FK (T -> R), depthwise along W with flipped FW, depthwise along H
 * with flipped FH, 1x1 by FC (R -> C). */
int cp4o_backward_data_unfused(const cp4o_shape* s, const float* dY,
                               const float* FK, const float* FC,
                               const float* FH, const float* FW, float* dX) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X, R = s->Rank, HW = H * W;
  int fail = 0;
#pragma omp parallel
  {
    float* a = (float*)malloc(sizeof(float) * (size_t)(R * HW));
    float* b = (float*)malloc(sizeof(float) * (size_t)(R * HW));
    if (!a || !b) {
#pragma omp atomic write
      fail = 1;
    }
#pragma omp for schedule(dynamic)
    for (long n = 0; n < N; ++n) {
      if (!a || !b) continue;
      pointwise_in(dY + n * T * HW, FK, a, T, R, HW);
      depthwise_h(a, FW, b, R, H, W, X, P, 1);
      depthwise_v(b, FH, a, R, H, W, Y, P, 1);
      pointwise_out(a, FC, dX + n * C * HW, C, R, HW);
    }
    free(a);
    free(b);
  }
  return fail;
}

/* Adjoint of depthwise_v / depthwise_h with unflipped taps:
 * dst[r,h,w] = sum_i F[i,r] src[r,h-i+P,w]  (resp. along W). */
static void depthwise_v_adj(const float* src, const float* F, float* dst,
                            long R, long H, long W, long Y, long P) {
  for (long r = 0; r < R; ++r)
    for (long h = 0; h < H; ++h) {
      float* dp = dst + (r * H + h) * W;
      memset(dp, 0, sizeof(float) * (size_t)W);
      for (long i = 0; i < Y; ++i) {
        const long hh = h - i + P;
        if (hh < 0 || hh >= H) continue;
        const float f = F[i * R + r];
        const float* sp = src + (r * H + hh) * W;
        for (long w = 0; w < W; ++w) dp[w] += f * sp[w];
      }
    }
}
static void depthwise_h_adj(const float* src, const float* F, float* dst,
                            long R, long H, long W, long X, long P) {
  for (long r = 0; r < R; ++r)
    for (long h = 0; h < H; ++h) {
      float* dp = dst + (r * H + h) * W;
      const float* sp = src + (r * H + h) * W;
      memset(dp, 0, sizeof(float) * (size_t)W);
      for (long j = 0; j < X; ++j) {
        const float f = F[j * R + r];
        for (long w = 0; w < W; ++w) {
          const long ww = w - j + P;
          if (ww >= 0 && ww < W) dp[w] += f * sp[ww];
        }
      }
    }
}

/* Factor gradients from the saved intermediates (double accumulators):
 *   A = FC^T x, B = FH *v A, Cc = FW *h B;  G3 = FK^T dy, G2 = adj_h(G3),
 *   G1 = adj_v(G2)
 *   dFK[t,r] = sum dy[n,t,p] Cc[n,r,p]        dFC[c,r] = sum x[n,c,p] G1[n,r,p]
 *   dFW[j,r] = sum G3[h,w] B[h,w+j-P]         dFH[i,r] = sum G2[h,w] A[h+i-P,w]
 * Outputs are overwritten.  These equal cp4Conv2dBackwardFilter.cu:64-257 by
 * reassociation of the sums. */
int cp4o_backward_filter_unfused(const cp4o_shape* s, const float* In,
                                 const float* dY, const float* FK,
                                 const float* FC, const float* FH,
                                 const float* FW, float* dFK, float* dFC,
                                 float* dFH, float* dFW) {
  const long N = s->N, H = s->H, W = s->W, P = s->pad, T = s->T, C = s->C,
             Y = s->Y, X = s->X, R = s->Rank, HW = H * W;
  const long nK = T * R, nC = C * R, nH = Y * R, nW = X * R;
  const long tot = nK + nC + nH + nW;
  double* acc = (double*)calloc((size_t)tot, sizeof(double));
  if (!acc) return 1;
  int fail = 0;
#pragma omp parallel
  {
    float* buf = (float*)malloc(sizeof(float) * (size_t)(6 * R * HW));
    double* loc = (double*)calloc((size_t)tot, sizeof(double));
    if (!buf || !loc) {
#pragma omp atomic write
      fail = 1;
    }
    float *A = buf, *B = buf + R * HW, *Cc = buf + 2 * R * HW,
          *G3 = buf + 3 * R * HW, *G2 = buf + 4 * R * HW, *G1 = buf + 5 * R * HW;
#pragma omp for schedule(dynamic)
    for (long n = 0; n < N; ++n) {
      if (!buf || !loc) continue;
      const float* xp = In + n * C * HW;
      const float* gp = dY + n * T * HW;
      pointwise_in(xp, FC, A, C, R, HW);
      depthwise_v(A, FH, B, R, H, W, Y, P, 0);
      depthwise_h(B, FW, Cc, R, H, W, X, P, 0);
      pointwise_in(gp, FK, G3, T, R, HW);
      depthwise_h_adj(G3, FW, G2, R, H, W, X, P);
      depthwise_v_adj(G2, FH, G1, R, H, W, Y, P);
      for (long t = 0; t < T; ++t)
        for (long r = 0; r < R; ++r) {
          double a = 0.0;
          for (long p = 0; p < HW; ++p) a += (double)gp[t * HW + p] * Cc[r * HW + p];
          loc[t * R + r] += a;
        }
      for (long c = 0; c < C; ++c)
        for (long r = 0; r < R; ++r) {
          double a = 0.0;
          for (long p = 0; p < HW; ++p) a += (double)xp[c * HW + p] * G1[r * HW + p];
          loc[nK + c * R + r] += a;
        }
      for (long i = 0; i < Y; ++i)
        for (long r = 0; r < R; ++r) {
          double a = 0.0;
          for (long h = 0; h < H; ++h) {
            const long hh = h + i - P;
            if (hh < 0 || hh >= H) continue;
            for (long w = 0; w < W; ++w)
              a += (double)G2[(r * H + h) * W + w] * A[(r * H + hh) * W + w];
          }
          loc[nK + nC + i * R + r] += a;
        }
      for (long j = 0; j < X; ++j)
        for (long r = 0; r < R; ++r) {
          double a = 0.0;
          for (long h = 0; h < H; ++h)
            for (long w = 0; w < W; ++w) {
              const long ww = w + j - P;
              if (ww >= 0 && ww < W)
                a += (double)G3[(r * H + h) * W + w] * B[(r * H + h) * W + ww];
            }
          loc[nK + nC + nH + j * R + r] += a;
        }
    }
#pragma omp critical
    {
      if (loc)
        for (long i = 0; i < tot; ++i) acc[i] += loc[i];
    }
    free(buf);
    free(loc);
  }
  for (long i = 0; i < nK; ++i) dFK[i] = (float)acc[i];
  for (long i = 0; i < nC; ++i) dFC[i] = (float)acc[nK + i];
  for (long i = 0; i < nH; ++i) dFH[i] = (float)acc[nK + nC + i];
  for (long i = 0; i < nW; ++i) dFW[i] = (float)acc[nK + nC + nH + i];
  free(acc);
  return fail;
}
