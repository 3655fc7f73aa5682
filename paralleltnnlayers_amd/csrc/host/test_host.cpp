// Host-API tests, the cases of the reference's doctest suite that concern this
// path (Cuda_kernels/test/test_Tensor.cpp.cu, test_Utils.cpp.cu,
// test_cp4Conv.cpp.cu) with a CPU dense convolution of the recomposed kernel
// standing in for cuDNN, plus the restored backward wrappers.  Needs a GPU.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <random>
#include <vector>

#include "bench_common.h"
#include "cp4/cp4conv2d.h"
#include "cp4/utils.h"

static int failures = 0;
#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::printf("CHECK failed: %s (%s:%d)\n", #cond, __FILE__, __LINE__); \
      ++failures;                                                          \
    }                                                                      \
  } while (0)

// Dense cross-correlation, H x W output, zero padding (what cuDNN computes
// for the reference's comparison when 2*pad == Y-1).
static Tensor dense_conv(Tensor const& In, Tensor const& K, unsigned pad) {
  const unsigned N = In.shape[0], C = In.shape[1], H = In.shape[2], W = In.shape[3];
  const unsigned T = K.shape[0], Y = K.shape[2], X = K.shape[3];
  Tensor Out{N, T, H, W};
  for (unsigned n = 0; n < N; ++n)
    for (unsigned t = 0; t < T; ++t)
      for (unsigned h = 0; h < H; ++h)
        for (unsigned w = 0; w < W; ++w) {
          double acc = 0;
          for (unsigned c = 0; c < C; ++c)
            for (unsigned y = 0; y < Y; ++y)
              for (unsigned x = 0; x < X; ++x) {
                const long hh = (long)h + y - pad, ww = (long)w + x - pad;
                if (hh < 0 || hh >= H || ww < 0 || ww >= W) continue;
                acc += (double)In.m_data[((n * C + c) * H + hh) * W + ww] *
                       K.m_data[((t * C + c) * Y + y) * X + x];
              }
          Out.m_data[((n * T + t) * H + h) * W + w] = (float)acc;
        }
  return Out;
}

static void test_tensor() {  // test_Tensor.cpp.cu:9-27
  std::mt19937 gen(7);
  std::uniform_real_distribution<> dis(-1.0, 1.0);
  Tensor ten = {40, 1, 1};
  for (size_t i = 0; i < ten.size(); ++i) CHECK(ten.m_data[i] == 0.f);  // zero-initialised
  for (size_t i = 0; i < ten.size(); ++i) ten.m_data[i] = (float)dis(gen);
  Tensor input(ten);
  CHECK(ten.size() == 40);
  CHECK(ten.order() == 3);
  for (size_t i = 0; i < ten.size(); ++i) CHECK(input.m_data[i] == ten.m_data[i]);
  Tensor other = {3, 2};
  other = ten;  // assignment also takes the shape
  CHECK(other.size() == 40 && other.shape.size() == 3 && other.m_data[7] == ten.m_data[7]);
  Tensor moved(std::move(other));
  CHECK(moved.size() == 40 && other.size() == 0);
  moved.upload();
  moved.m_data[0] = 123.f;
  moved.download();
  CHECK(moved.m_data[0] == ten.m_data[0]);  // round trip through HBM
  tensor_shape a, b;
  a.N = 1; b.N = 1; a.Rank = 2; b.Rank = 3;
  CHECK(a < b && !(b < a));
}

static void test_utils() {  // test_Utils.cpp.cu:10-51
  Tensor K0 = random_fill({16, 6}), K1 = random_fill({16, 6});
  Tensor K2 = random_fill({3, 6}), K3 = random_fill({3, 6});
  Tensor U = random_fill({1, 16, 32, 32});
  for (size_t i = 0; i < U.size(); ++i) CHECK(U.m_data[i] > 0 && U.m_data[i] <= 1.f);
  CHECK(K0.m_data[5] == K1.m_data[5]);  // same seed, same stream prefix
  Tensor K = cp4recom(K0, K1, K2, K3);
  CHECK(K.size() == 2304 && K.order() == 4);
  CHECK(K.shape[0] == 16 && K.shape[1] == 16 && K.shape[2] == 3 && K.shape[3] == 3);
  Tensor V = CP::Conv2dForward(U, K0, K1, K2, K3, 1);
  Tensor V2 = CP::Conv2dForward(U, K0, K1, K2, K3, 1);
  CHECK(V.size() == 1 * 16 * 32 * 32 && V.order() == 4);
  CHECK(V.shape[0] == 1 && V.shape[1] == 16 && V.shape[2] == 32 && V.shape[3] == 32);
  for (size_t i = 0; i < V.size(); ++i) CHECK(V.m_data[i] != 0);
  CHECK(AllClose(V, V2, 1e-5f));
  Tensor D = dense_conv(U, K, 1);
  CHECK(AllClose(D, V, 1e-4f));
  V.m_data[0] *= 2;
  CHECK(!AllClose(V, V2, 1e-1f));
}

static void test_conv_passes() {  // test_cp4Conv.cpp.cu:14-101, smaller shape
  const unsigned n = 2, c = 6, x = 13, pad = 2, t = 8, f = 5, rank = 4;
  Tensor Input = random_fill({n, c, x, x}), dV = random_fill({n, t, x, x});
  Tensor FT = random_fill({t, rank}), FC = random_fill({c, rank});
  Tensor FY = random_fill({f, rank}), FX = random_fill({f, rank});
  // decorrelate the identical random streams a little
  for (size_t i = 0; i < dV.size(); ++i) dV.m_data[i] = 1.f - 0.5f * dV.m_data[i];
  for (size_t i = 0; i < FC.size(); ++i) FC.m_data[i] = 0.25f + FC.m_data[i] * FC.m_data[i];
  Tensor K = cp4recom(FT, FC, FY, FX);
  Tensor Dense = dense_conv(Input, K, pad);
  Tensor CP4 = CP::Conv2dForward(Input, FT, FC, FY, FX, pad);
  CHECK(CP4.shape[0] == n && CP4.shape[1] == t && CP4.shape[2] == x && CP4.shape[3] == x);
  CHECK(AllClose(Dense, CP4, 1e-4f));
  // backward-data: adjoint identity <y, dV> == <Input, dX>
  Tensor dX = CP::Conv2dBackwardData(dV, FT, FC, FY, FX, pad);
  CHECK(dX.shape[0] == n && dX.shape[1] == c && dX.shape[2] == x && dX.shape[3] == x);
  double lhs = 0, rhs = 0;
  for (size_t i = 0; i < CP4.size(); ++i) lhs += (double)CP4.m_data[i] * dV.m_data[i];
  for (size_t i = 0; i < dX.size(); ++i) rhs += (double)dX.m_data[i] * Input.m_data[i];
  CHECK(std::fabs(lhs - rhs) <= 1e-4 * std::fabs(lhs));
  // backward-filter: dFT contracts the dense gradient with the other factors
  auto g = CP::Conv2dBackwardFilter(dV, Input, FT, FC, FY, FX, pad);
  CHECK(g.dFT.shape[0] == t && g.dFT.shape[1] == rank && g.dFX.shape[0] == f);
  Tensor FF{t, c, f, f};
  cp4_conv2d_backward_filter_full_gpu({n, x, x, pad, t, c, f, f, rank}, FF.m_data, Input.m_data,
                                      dV.m_data);
  Tensor want{t, rank};
  for (unsigned tt = 0; tt < t; ++tt)
    for (unsigned r = 0; r < rank; ++r) {
      double acc = 0;
      for (unsigned cc = 0; cc < c; ++cc)
        for (unsigned y = 0; y < f; ++y)
          for (unsigned xx = 0; xx < f; ++xx)
            acc += (double)FF.m_data[((tt * c + cc) * f + y) * f + xx] * FC.m_data[cc * rank + r] *
                   FY.m_data[y * rank + r] * FX.m_data[xx * rank + r];
      want.m_data[tt * rank + r] = (float)acc;
    }
  CHECK(AllClose(want, g.dFT, 1e-3f));
  // the per-factor launcher ADDS into its output (cp4Conv2dBackwardFilter.cu:99)
  Tensor acc{t, rank};
  for (size_t i = 0; i < acc.size(); ++i) acc.m_data[i] = 1.f;
  cp4_conv2d_backward_filter_t_gpu({n, x, x, pad, t, c, f, f, rank}, acc.m_data, Input.m_data,
                                   dV.m_data, FC.m_data, FY.m_data, FX.m_data);
  for (size_t i = 0; i < acc.size(); ++i) acc.m_data[i] -= 1.f;
  CHECK(AllClose(acc, g.dFT, 1e-3f));
}

static void test_shape_list() {  // BenchBothTime.cu:14-25, 59-82
  const char* path = "cp4_host_test_shapes.txt";
  {
    std::ofstream f(path);
    f << "# comment\n\n1   3 224 224 5    96 11 11\n1  48  55  55 2   256  5  5\n"
      << "1 3 224 224 5 96 11 11\n";
  }
  std::vector<tensor_shape> shapes;
  CHECK(read_shapes(path, &shapes));
  CHECK(shapes.size() == 2 && shapes[0].T == 96 && shapes[1].C == 48 && shapes[1].pad == 2);
  std::remove(path);
  tensor_shape p = shapes[1];
  p.Rank = 4;
  auto r = CP::run_convolution(p, 3);
  CHECK(r.first > 0.f);
  CHECK(r.second == 4u * (1 * 256 * 55 * 55 + 1 * 48 * 55 * 55 + 4 * (256 + 48 + 5 + 5)));
}

int main() {
  test_tensor();
  test_utils();
  test_conv_passes();
  test_shape_list();
  if (failures) {
    std::printf("%d host API checks failed\n", failures);
    return 1;
  }
  std::printf("host API tests passed\n");
  return 0;
}
