// namespace CP and the raw-pointer launchers of the reference, on the C ABI.
#include "cp4/cp4conv2d.h"

#include <cstdio>
#include <cstdlib>
#include <memory>
#include <vector>

#include "cp4/capi.h"

namespace {

[[noreturn]] void die(cp4_status st, const char* where) {
  // the reference prints and exits on any runtime error
  // (Cuda_kernels/cp4Conv2dForward.cu:10-19)
  std::fprintf(stderr, "cp4 assert: %s (%s) in %s\n", cp4_status_string(st),
               cp4_last_error_message(), where);
  std::exit((int)st);
}
void check(cp4_status st, const char* where) {
  if (st != CP4_OK) die(st, where);
}

cp4_shape to_c(const tensor_shape& p) {
  return cp4_shape{p.N, p.H, p.W, p.pad, p.T, p.C, p.Y, p.X, p.Rank};
}

// A device view of a caller buffer that may live in host or device memory.
// Host data is staged into a temporary HBM buffer (and copied back if written).
class DeviceView {
 public:
  DeviceView(const float* p, size_t n, bool is_input, bool is_output)
      : host_(nullptr), dev_(const_cast<float*>(p)), n_(n), out_(is_output), owned_(false) {
    if (!p || n == 0) return;
    int is_dev = 0;
    check(cp4_pointer_is_device(p, &is_dev), "pointer query");
    if (is_dev) return;
    host_ = const_cast<float*>(p);
    void* d = nullptr;
    check(cp4_device_malloc(&d, n * sizeof(float)), "staging allocation");
    dev_ = static_cast<float*>(d);
    owned_ = true;
    if (is_input) check(cp4_memcpy_h2d(dev_, host_, n * sizeof(float), nullptr), "staging upload");
  }
  ~DeviceView() {
    if (!owned_) return;
    if (out_) {
      check(cp4_memcpy_d2h(host_, dev_, n_ * sizeof(float), nullptr), "staging download");
      check(cp4_stream_synchronize(nullptr), "staging sync");
    }
    check(cp4_device_free(dev_), "staging free");
  }
  DeviceView(const DeviceView&) = delete;
  DeviceView& operator=(const DeviceView&) = delete;
  float* get() const { return dev_; }

 private:
  float* host_;
  float* dev_;
  size_t n_;
  bool out_, owned_;
};

size_t in_elems(const tensor_shape& p) { return (size_t)p.N * p.C * p.H * p.W; }
size_t out_elems(const tensor_shape& p) { return (size_t)p.N * p.T * p.H * p.W; }

// One factor gradient through the fused call.  `which` names the wanted
// gradient (0 T, 1 C, 2 Y, 3 X); its own factor does not enter its gradient,
// so a zero matrix stands in for it.  The result is ADDED into `out`.
float filter_factor(tensor_shape p, int which, float* out, const float* In, const float* dLdO,
                    const float* f0, const float* f1, const float* f2) {
  const cp4_shape s = to_c(p);
  const size_t dims[4] = {p.T, p.C, p.Y, p.X};
  const float* given[3] = {f0, f1, f2};
  DeviceView x(In, in_elems(p), true, false), dy(dLdO, out_elems(p), true, false);
  std::vector<std::unique_ptr<DeviceView>> views;
  float* fac[4];
  void* grads[4];
  void* dummy = nullptr;
  int g = 0;
  for (int i = 0; i < 4; ++i) {
    const size_t n = dims[i] * p.Rank;
    check(cp4_device_malloc(&grads[i], n * sizeof(float)), "gradient allocation");
    if (i == which) {
      check(cp4_device_malloc(&dummy, n * sizeof(float)), "factor allocation");
      check(cp4_memset_zero(dummy, n * sizeof(float), nullptr), "factor clear");
      fac[i] = static_cast<float*>(dummy);
    } else {
      views.emplace_back(new DeviceView(given[g++], n, true, false));
      fac[i] = views.back()->get();
    }
  }
  const size_t ws_bytes = cp4_conv2d_backward_filter_workspace_bytes(&s);
  void* ws = nullptr;
  check(cp4_device_malloc(&ws, ws_bytes), "workspace allocation");
  check(cp4_conv2d_backward_filter(&s, x.get(), dy.get(), fac[0], fac[1], fac[2], fac[3],
                                   (float*)grads[0], (float*)grads[1], (float*)grads[2],
                                   (float*)grads[3], ws, ws_bytes, nullptr),
        "cp4_conv2d_backward_filter");
  // out += gradient, on the host side of whatever memory `out` is
  const size_t n = dims[which] * p.Rank;
  std::vector<float> gh(n), oh(n);
  check(cp4_memcpy_d2h(gh.data(), grads[which], n * sizeof(float), nullptr), "gradient download");
  check(cp4_stream_synchronize(nullptr), "sync");
  int out_dev = 0;
  check(cp4_pointer_is_device(out, &out_dev), "pointer query");
  if (out_dev) {
    check(cp4_memcpy_d2h(oh.data(), out, n * sizeof(float), nullptr), "output download");
    check(cp4_stream_synchronize(nullptr), "sync");
    for (size_t i = 0; i < n; ++i) oh[i] += gh[i];
    check(cp4_memcpy_h2d(out, oh.data(), n * sizeof(float), nullptr), "output upload");
    check(cp4_stream_synchronize(nullptr), "sync");
  } else {
    for (size_t i = 0; i < n; ++i) out[i] += gh[i];
  }
  for (int i = 0; i < 4; ++i) check(cp4_device_free(grads[i]), "free");
  check(cp4_device_free(dummy), "free");
  check(cp4_device_free(ws), "free");
  return 0.f;  // the reference's host loops return 0 as well
}

}  // namespace

float cp4_conv2d_forward_gpu(tensor_shape p, const float* In, const float* FT, const float* FC,
                             const float* FY, const float* FX, float* Out, unsigned PROFCOUNT) {
  if (p.Y != p.X)  // the reference only warns (cp4Conv2dForward.cu:206); so do we
    std::fprintf(stderr, "Invalid filter shape. Height must equal width\n");
  const cp4_shape s = to_c(p);
  DeviceView x(In, in_elems(p), true, false), y(Out, out_elems(p), false, true);
  DeviceView ft(FT, (size_t)p.T * p.Rank, true, false), fc(FC, (size_t)p.C * p.Rank, true, false);
  DeviceView fy(FY, (size_t)p.Y * p.Rank, true, false), fx(FX, (size_t)p.X * p.Rank, true, false);
  float us = 0.f;
  check(cp4_time_forward(&s, x.get(), ft.get(), fc.get(), fy.get(), fx.get(), y.get(), 0,
                         PROFCOUNT ? PROFCOUNT : 1, &us, nullptr),
        "cp4_conv2d_forward_gpu");
  return us;
}

float cp4_conv2d_backward_data_gpu(tensor_shape p, const float* Up, const float* FT,
                                   const float* FC, const float* FY, const float* FX, float* Out,
                                   unsigned PROFCOUNT) {
  if (p.Y != p.X) std::fprintf(stderr, "Invalid filter shape. Height must equal width\n");
  const cp4_shape s = to_c(p);
  DeviceView dy(Up, out_elems(p), true, false), dx(Out, in_elems(p), false, true);
  DeviceView ft(FT, (size_t)p.T * p.Rank, true, false), fc(FC, (size_t)p.C * p.Rank, true, false);
  DeviceView fy(FY, (size_t)p.Y * p.Rank, true, false), fx(FX, (size_t)p.X * p.Rank, true, false);
  float us = 0.f;
  check(cp4_time_backward_data(&s, dy.get(), ft.get(), fc.get(), fy.get(), fx.get(), dx.get(), 0,
                               PROFCOUNT ? PROFCOUNT : 1, &us, nullptr),
        "cp4_conv2d_backward_data_gpu");
  return us;
}

float cp4_conv2d_backward_filter_full_gpu(tensor_shape p, float* FF, const float* In,
                                          const float* dLdO, unsigned) {
  const cp4_shape s = to_c(p);
  DeviceView x(In, in_elems(p), true, false), dy(dLdO, out_elems(p), true, false);
  DeviceView ff(FF, (size_t)p.T * p.C * p.Y * p.X, true, true);
  check(cp4_conv2d_backward_filter_full(&s, x.get(), dy.get(), ff.get(), 1, nullptr),
        "cp4_conv2d_backward_filter_full_gpu");
  check(cp4_stream_synchronize(nullptr), "sync");
  return 0.f;
}

float cp4_conv2d_backward_filter_t_gpu(tensor_shape p, float* dFT, const float* In,
                                       const float* dLdO, const float* FC, const float* FY,
                                       const float* FX, unsigned) {
  return filter_factor(p, 0, dFT, In, dLdO, FC, FY, FX);
}
float cp4_conv2d_backward_filter_c_gpu(tensor_shape p, float* dFC, const float* In,
                                       const float* dLdO, const float* FT, const float* FY,
                                       const float* FX, unsigned) {
  return filter_factor(p, 1, dFC, In, dLdO, FT, FY, FX);
}
float cp4_conv2d_backward_filter_y_gpu(tensor_shape p, float* dFY, const float* In,
                                       const float* dLdO, const float* FT, const float* FC,
                                       const float* FX, unsigned) {
  return filter_factor(p, 2, dFY, In, dLdO, FT, FC, FX);
}
float cp4_conv2d_backward_filter_x_gpu(tensor_shape p, float* dFX, const float* In,
                                       const float* dLdO, const float* FT, const float* FC,
                                       const float* FY, unsigned) {
  return filter_factor(p, 3, dFX, In, dLdO, FT, FC, FY);
}

namespace CP {

Tensor Conv2dForward(Tensor const& Input, Tensor const& FT, Tensor const& FC, Tensor const& FY,
                     Tensor const& FX, unsigned pad) {
  tensor_shape p;  // cp4Conv2d.cu:21-30
  p.N = Input.shape[0];
  p.C = Input.shape[1];
  p.H = Input.shape[2];
  p.W = Input.shape[3];
  p.pad = pad;
  p.Rank = FT.shape[1];
  p.T = FT.shape[0];
  p.Y = FY.shape[0];
  p.X = FX.shape[0];
  Tensor Out{p.N, p.T, p.H, p.W};
  for (const Tensor* t : {&Input, &FT, &FC, &FY, &FX}) t->upload();
  cp4_conv2d_forward_gpu(p, Input.device(), FT.device(), FC.device(), FY.device(), FX.device(),
                         Out.device());
  Out.download();
  return Out;
}

Tensor Conv2dBackwardData(Tensor const& Up, Tensor const& FT, Tensor const& FC, Tensor const& FY,
                          Tensor const& FX, unsigned pad) {
  tensor_shape p;  // cp4Conv2d.cu:55-64
  p.N = Up.shape[0];
  p.T = Up.shape[1];
  p.H = Up.shape[2];
  p.W = Up.shape[3];
  p.pad = pad;
  p.Rank = FT.shape[1];
  p.C = FC.shape[0];
  p.Y = FY.shape[0];
  p.X = FX.shape[0];
  Tensor Out{p.N, p.C, p.H, p.W};
  for (const Tensor* t : {&Up, &FT, &FC, &FY, &FX}) t->upload();
  cp4_conv2d_backward_data_gpu(p, Up.device(), FT.device(), FC.device(), FY.device(),
                               FX.device(), Out.device());
  Out.download();
  return Out;
}

FilterGradients Conv2dBackwardFilter(Tensor const& dLdO, Tensor const& In, Tensor const& FT,
                                     Tensor const& FC, Tensor const& FY, Tensor const& FX,
                                     unsigned pad) {
  tensor_shape p;  // cp4Conv2d.cu:91-100
  p.N = dLdO.shape[0];
  p.T = dLdO.shape[1];
  p.H = dLdO.shape[2];
  p.W = dLdO.shape[3];
  p.pad = pad;
  p.Rank = FT.shape[1];
  p.C = FC.shape[0];
  p.Y = FY.shape[0];
  p.X = FX.shape[0];
  FilterGradients g{Tensor{p.T, p.Rank}, Tensor{p.C, p.Rank}, Tensor{p.Y, p.Rank},
                    Tensor{p.X, p.Rank}};
  for (const Tensor* t : {&dLdO, &In, &FT, &FC, &FY, &FX}) t->upload();
  const cp4_shape s = to_c(p);
  const size_t ws_bytes = cp4_conv2d_backward_filter_workspace_bytes(&s);
  void* ws = nullptr;
  check(cp4_device_malloc(&ws, ws_bytes), "workspace allocation");
  check(cp4_conv2d_backward_filter(&s, In.device(), dLdO.device(), FT.device(), FC.device(),
                                   FY.device(), FX.device(), g.dFT.device(), g.dFC.device(),
                                   g.dFY.device(), g.dFX.device(), ws, ws_bytes, nullptr),
        "CP::Conv2dBackwardFilter");
  g.dFT.download();
  g.dFC.download();
  g.dFY.download();
  g.dFX.download();
  check(cp4_device_free(ws), "workspace free");
  return g;
}

std::pair<float, unsigned> run_convolution(tensor_shape p, unsigned PROFCOUNT) {
  void* buf[6];
  const size_t n[6] = {in_elems(p),           (size_t)p.T * p.Rank, (size_t)p.C * p.Rank,
                       (size_t)p.Y * p.Rank, (size_t)p.X * p.Rank, out_elems(p)};
  for (int i = 0; i < 6; ++i) check(cp4_device_malloc(&buf[i], n[i] * sizeof(float)), "allocation");
  const unsigned mem = (unsigned)(sizeof(float) * ((size_t)p.N * p.T * p.H * p.W +
                                                   (size_t)p.N * p.C * p.H * p.W +
                                                   (size_t)p.Rank * (p.T + p.C + p.X + p.Y)));
  // one untimed launch first: the first use of a kernel loads its code object
  // (about a millisecond), which is not launch time
  (void)cp4_conv2d_forward_gpu(p, (float*)buf[0], (float*)buf[1], (float*)buf[2], (float*)buf[3],
                               (float*)buf[4], (float*)buf[5], 1);
  const float us =
      cp4_conv2d_forward_gpu(p, (float*)buf[0], (float*)buf[1], (float*)buf[2], (float*)buf[3],
                             (float*)buf[4], (float*)buf[5], PROFCOUNT);
  for (int i = 0; i < 6; ++i) check(cp4_device_free(buf[i]), "free");
  return std::make_pair(us, mem);
}

}  // namespace CP
