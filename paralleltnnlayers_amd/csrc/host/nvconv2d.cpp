// namespace NV over the C ABI of the dense comparator (include/cp4/dense.h).
// Mirrors Cuda_kernels/NVConv2d.cu:154-171, 296-314, 439-461, 471-489.
#include "cp4/nvconv2d.h"

#include <cstdio>
#include <cstdlib>

#include "cp4/dense.h"

namespace {

// The reference prints the library's error and exits (NVConv2d.cu:9-16).
void check(cp4_status st, const char* where) {
  if (st == CP4_OK) return;
  std::fprintf(stderr, "Error in %s: %s (%s %s)\n", where, cp4_status_string(st),
               cp4_dense_last_error_message(), cp4_last_error_message());
  std::exit(EXIT_FAILURE);
}

cp4_shape shape_of(unsigned N, unsigned C, unsigned H, unsigned W, unsigned pad, Tensor const& K) {
  return cp4_shape{N, H, W, pad, K.shape[0], C, K.shape[2], K.shape[3], 0};
}

void need(bool ok, const char* what) {
  if (ok) return;
  std::fprintf(stderr, "NV: %s\n", what);
  std::exit(EXIT_FAILURE);
}

}  // namespace

namespace NV {

Tensor Conv2dForward(Tensor const& In, Tensor const& K, unsigned pad) {
  need(In.order() == 4 && K.order() == 4 && In.shape[1] == K.shape[1], "Conv2dForward: shapes");
  const cp4_shape s = shape_of(In.shape[0], In.shape[1], In.shape[2], In.shape[3], pad, K);
  Tensor V({s.N, s.T, s.H, s.W});
  In.upload();
  K.upload();
  check(cp4_dense_conv2d_forward(&s, In.device(), K.device(), V.device(), nullptr),
        "NV::Conv2dForward");
  V.download();
  return V;
}

Tensor Conv2dBackwardData(Tensor const& Upstream, Tensor const& K, unsigned pad) {
  need(Upstream.order() == 4 && K.order() == 4 && Upstream.shape[1] == K.shape[0],
       "Conv2dBackwardData: shapes");
  const cp4_shape s =
      shape_of(Upstream.shape[0], K.shape[1], Upstream.shape[2], Upstream.shape[3], pad, K);
  Tensor V({s.N, s.C, s.H, s.W});
  Upstream.upload();
  K.upload();
  check(cp4_dense_conv2d_backward_data(&s, Upstream.device(), K.device(), V.device(), nullptr),
        "NV::Conv2dBackwardData");
  V.download();
  return V;
}

Tensor Conv2dBackwardFilter(Tensor const& dLdO, Tensor const& Input, Tensor const& Filter,
                            unsigned pad) {
  need(dLdO.order() == 4 && Input.order() == 4 && Filter.order() == 4 &&
           Input.shape[1] == Filter.shape[1] && dLdO.shape[1] == Filter.shape[0],
       "Conv2dBackwardFilter: shapes");
  const cp4_shape s =
      shape_of(Input.shape[0], Input.shape[1], Input.shape[2], Input.shape[3], pad, Filter);
  Tensor V({s.T, s.C, s.Y, s.X});
  dLdO.upload();
  Input.upload();
  check(cp4_dense_conv2d_backward_filter(&s, Input.device(), dLdO.device(), V.device(), nullptr),
        "NV::Conv2dBackwardFilter");
  V.download();
  return V;
}

std::pair<float, unsigned> run_convolution(tensor_shape p, unsigned PROFCOUNT) {
  const cp4_shape s{p.N, p.H, p.W, p.pad, p.T, p.C, p.Y, p.X, 0};
  const size_t n[3] = {(size_t)p.N * p.C * p.H * p.W, (size_t)p.T * p.C * p.Y * p.X,
                       (size_t)p.N * p.T * p.H * p.W};
  void* buf[3];
  for (int i = 0; i < 3; ++i)
    check(cp4_device_malloc(&buf[i], n[i] * sizeof(float)), "NV::run_convolution allocation");
  float us = 0.f;
  check(cp4_dense_time_forward(&s, (float*)buf[0], (float*)buf[1], (float*)buf[2], 0,
                               PROFCOUNT ? PROFCOUNT : 1, &us, nullptr),
        "NV::run_convolution");
  for (int i = 0; i < 3; ++i) check(cp4_device_free(buf[i]), "NV::run_convolution free");
  const unsigned mem = (unsigned)(sizeof(float) * (n[0] + n[1] + n[2]));
  return std::make_pair(us, mem);
}

}  // namespace NV
