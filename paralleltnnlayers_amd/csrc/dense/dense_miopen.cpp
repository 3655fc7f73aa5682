// Dense-convolution comparator over MIOpen (immediate mode): the vendor
// library's fp32 NCHW convolution behind the C ABI of include/cp4/dense.h.
// Stands where the reference calls cuDNN (Cuda_kernels/NVConv2d.cu:18-433).
//
// One library handle per process; per problem (shape, direction) the fastest
// applicable solution is looked up once, compiled, and cached with its
// workspace.  Calls are serialised by one mutex: this is a comparator, not a
// hot path.
#include <hip/hip_runtime.h>
#include <miopen/miopen.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "cp4/dense.h"

namespace {

thread_local std::string g_err;

cp4_status fail(cp4_status s, const std::string& msg) {
  g_err = msg;
  return s;
}

#define DENSE_MIOPEN(call)                                                              \
  do {                                                                                  \
    miopenStatus_t st_ = (call);                                                        \
    if (st_ != miopenStatusSuccess)                                                     \
      return fail(CP4_ERR_HIP, std::string(#call) + ": " + miopenGetErrorString(st_));  \
  } while (0)
#define DENSE_HIP(call)                                                                 \
  do {                                                                                  \
    hipError_t e_ = (call);                                                             \
    if (e_ != hipSuccess)                                                               \
      return fail(CP4_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(e_));      \
  } while (0)

enum Dir { kFwd = 0, kBwdData = 1, kBwdFilter = 2 };

struct Problem {
  miopenTensorDescriptor_t x = nullptr, w = nullptr, y = nullptr;
  miopenConvolutionDescriptor_t conv = nullptr;
  bool have[3] = {false, false, false};
  uint64_t solution[3] = {0, 0, 0};
  size_t ws_bytes[3] = {0, 0, 0};
};

using Key = std::tuple<unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned,
                       unsigned>;

std::mutex g_mu;
miopenHandle_t g_handle = nullptr;
std::map<Key, Problem> g_problems;
void* g_ws = nullptr;
size_t g_ws_cap = 0;

cp4_status check(const cp4_shape* s) {
  if (!s) return fail(CP4_ERR_NULL_POINTER, "shape is null");
  if (!s->N || !s->C || !s->H || !s->W || !s->T || !s->Y || !s->X)
    return fail(CP4_ERR_SHAPE, "a dimension is zero");
  if (2 * s->pad + 1 != s->Y || 2 * s->pad + 1 != s->X)
    return fail(CP4_ERR_SHAPE,
                "the dense comparator needs 2*pad = Y-1 = X-1 (H x W output of the library)");
  return CP4_OK;
}

cp4_status get_problem(const cp4_shape& s, Problem** out) {
  if (!g_handle) {
    // MIOpen keeps its kernel cache under the home directory; fall back to a
    // per-user directory in /tmp where the caller has not chosen a place.
    if (!getenv("MIOPEN_USER_DB_PATH") && !getenv("HOME")) {
      static std::string dir = "/tmp/cp4_miopen_" + std::to_string((unsigned)getuid());
      setenv("MIOPEN_USER_DB_PATH", dir.c_str(), 0);
    }
    DENSE_MIOPEN(miopenCreate(&g_handle));
  }
  const Key k(s.N, s.C, s.H, s.W, s.pad, s.T, s.Y, s.X);
  auto it = g_problems.find(k);
  if (it == g_problems.end()) {
    Problem p;
    DENSE_MIOPEN(miopenCreateTensorDescriptor(&p.x));
    DENSE_MIOPEN(miopenSet4dTensorDescriptor(p.x, miopenFloat, (int)s.N, (int)s.C, (int)s.H,
                                             (int)s.W));
    DENSE_MIOPEN(miopenCreateTensorDescriptor(&p.w));
    DENSE_MIOPEN(miopenSet4dTensorDescriptor(p.w, miopenFloat, (int)s.T, (int)s.C, (int)s.Y,
                                             (int)s.X));
    DENSE_MIOPEN(miopenCreateTensorDescriptor(&p.y));
    DENSE_MIOPEN(miopenSet4dTensorDescriptor(p.y, miopenFloat, (int)s.N, (int)s.T, (int)s.H,
                                             (int)s.W));
    DENSE_MIOPEN(miopenCreateConvolutionDescriptor(&p.conv));
    // cross-correlation, as CUDNN_CROSS_CORRELATION in NVConv2d.cu:57-66
    DENSE_MIOPEN(miopenInitConvolutionDescriptor(p.conv, miopenConvolution, (int)s.pad,
                                                 (int)s.pad, 1, 1, 1, 1));
    int n, c, h, w;
    DENSE_MIOPEN(miopenGetConvolutionForwardOutputDim(p.conv, p.x, p.w, &n, &c, &h, &w));
    if (n != (int)s.N || c != (int)s.T || h != (int)s.H || w != (int)s.W)
      return fail(CP4_ERR_SHAPE, "library output size differs from [N,T,H,W]");
    it = g_problems.emplace(k, p).first;
  }
  *out = &it->second;
  return CP4_OK;
}

// Picks, compiles and remembers the fastest solution of one direction.
cp4_status prepare(Problem& p, Dir d) {
  if (p.have[d]) return CP4_OK;
  size_t count = 0;
  switch (d) {
    case kFwd:
      DENSE_MIOPEN(miopenConvolutionForwardGetSolutionCount(g_handle, p.w, p.x, p.conv, p.y,
                                                            &count));
      break;
    case kBwdData:
      DENSE_MIOPEN(miopenConvolutionBackwardDataGetSolutionCount(g_handle, p.y, p.w, p.conv,
                                                                 p.x, &count));
      break;
    default:
      DENSE_MIOPEN(miopenConvolutionBackwardWeightsGetSolutionCount(g_handle, p.y, p.x, p.conv,
                                                                    p.w, &count));
  }
  if (count == 0) return fail(CP4_ERR_UNSUPPORTED, "the library offers no solution");
  std::vector<miopenConvSolution_t> sol(count);
  size_t got = 0;
  switch (d) {
    case kFwd:
      DENSE_MIOPEN(miopenConvolutionForwardGetSolution(g_handle, p.w, p.x, p.conv, p.y, count,
                                                       &got, sol.data()));
      break;
    case kBwdData:
      DENSE_MIOPEN(miopenConvolutionBackwardDataGetSolution(g_handle, p.y, p.w, p.conv, p.x,
                                                            count, &got, sol.data()));
      break;
    default:
      DENSE_MIOPEN(miopenConvolutionBackwardWeightsGetSolution(g_handle, p.y, p.x, p.conv, p.w,
                                                               count, &got, sol.data()));
  }
  if (got == 0) return fail(CP4_ERR_UNSUPPORTED, "the library returned no solution");
  // the list comes sorted by expected time, fastest first
  const miopenConvSolution_t best = sol[0];
  switch (d) {
    case kFwd:
      DENSE_MIOPEN(miopenConvolutionForwardCompileSolution(g_handle, p.w, p.x, p.conv, p.y,
                                                           best.solution_id));
      break;
    case kBwdData:
      DENSE_MIOPEN(miopenConvolutionBackwardDataCompileSolution(g_handle, p.y, p.w, p.conv, p.x,
                                                                best.solution_id));
      break;
    default:
      DENSE_MIOPEN(miopenConvolutionBackwardWeightsCompileSolution(g_handle, p.y, p.x, p.conv,
                                                                   p.w, best.solution_id));
  }
  p.solution[d] = best.solution_id;
  p.ws_bytes[d] = best.workspace_size;
  p.have[d] = true;
  return CP4_OK;
}

cp4_status workspace(size_t bytes) {
  if (bytes <= g_ws_cap) return CP4_OK;
  if (g_ws) DENSE_HIP(hipFree(g_ws));
  g_ws = nullptr;
  g_ws_cap = 0;
  DENSE_HIP(hipMalloc(&g_ws, bytes));
  g_ws_cap = bytes;
  return CP4_OK;
}

cp4_status run(const cp4_shape* s, Dir d, const void* a, const void* b, void* out,
               cp4_stream stream) {
  cp4_status rc = check(s);
  if (rc != CP4_OK) return rc;
  if (!a || !b || !out) return fail(CP4_ERR_NULL_POINTER, "a data pointer is null");
  Problem* p = nullptr;
  rc = get_problem(*s, &p);
  if (rc != CP4_OK) return rc;
  DENSE_MIOPEN(miopenSetStream(g_handle, static_cast<hipStream_t>(stream)));
  rc = prepare(*p, d);
  if (rc != CP4_OK) return rc;
  rc = workspace(p->ws_bytes[d]);
  if (rc != CP4_OK) return rc;
  void* ws = p->ws_bytes[d] ? g_ws : nullptr;
  switch (d) {
    case kFwd:   // a = x, b = K, out = y
      DENSE_MIOPEN(miopenConvolutionForwardImmediate(g_handle, p->w, b, p->x, a, p->conv, p->y,
                                                     out, ws, p->ws_bytes[d], p->solution[d]));
      break;
    case kBwdData:   // a = dy, b = K, out = dx
      DENSE_MIOPEN(miopenConvolutionBackwardDataImmediate(g_handle, p->y, a, p->w, b, p->conv,
                                                          p->x, out, ws, p->ws_bytes[d],
                                                          p->solution[d]));
      break;
    default:   // a = x, b = dy, out = dK
      DENSE_MIOPEN(miopenConvolutionBackwardWeightsImmediate(g_handle, p->y, b, p->x, a, p->conv,
                                                             p->w, out, ws, p->ws_bytes[d],
                                                             p->solution[d]));
  }
  return CP4_OK;
}

}  // namespace

extern "C" {

const char* cp4_dense_last_error_message(void) { return g_err.c_str(); }

cp4_status cp4_dense_conv2d_forward(const cp4_shape* shape, const float* x, const float* K,
                                    float* y, cp4_stream stream) {
  std::lock_guard<std::mutex> lk(g_mu);
  return run(shape, kFwd, x, K, y, stream);
}

cp4_status cp4_dense_conv2d_backward_data(const cp4_shape* shape, const float* dy,
                                          const float* K, float* dx, cp4_stream stream) {
  std::lock_guard<std::mutex> lk(g_mu);
  return run(shape, kBwdData, dy, K, dx, stream);
}

cp4_status cp4_dense_conv2d_backward_filter(const cp4_shape* shape, const float* x,
                                            const float* dy, float* dK, cp4_stream stream) {
  std::lock_guard<std::mutex> lk(g_mu);
  return run(shape, kBwdFilter, x, dy, dK, stream);
}

cp4_status cp4_dense_time_forward(const cp4_shape* shape, const float* x, const float* K,
                                  float* y, unsigned warmup, unsigned profcount, float* mean_us,
                                  cp4_stream stream) {
  if (!mean_us) return fail(CP4_ERR_NULL_POINTER, "mean_us is null");
  if (profcount == 0) return fail(CP4_ERR_SHAPE, "profcount is zero");
  std::lock_guard<std::mutex> lk(g_mu);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // the first call looks the solution up and compiles it: never timed
  cp4_status rc = run(shape, kFwd, x, K, y, stream);
  for (unsigned i = 0; rc == CP4_OK && i < warmup; ++i) rc = run(shape, kFwd, x, K, y, stream);
  if (rc != CP4_OK) return rc;
  hipEvent_t e0, e1;
  DENSE_HIP(hipEventCreate(&e0));
  DENSE_HIP(hipEventCreate(&e1));
  DENSE_HIP(hipEventRecord(e0, st));
  for (unsigned i = 0; rc == CP4_OK && i < profcount; ++i) rc = run(shape, kFwd, x, K, y, stream);
  DENSE_HIP(hipEventRecord(e1, st));
  DENSE_HIP(hipEventSynchronize(e1));
  float ms = 0.f;
  DENSE_HIP(hipEventElapsedTime(&ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != CP4_OK) return rc;
  *mean_us = ms * 1000.f / (float)profcount;
  return CP4_OK;
}

void cp4_dense_release(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  for (auto& kv : g_problems) {
    Problem& p = kv.second;
    if (p.x) miopenDestroyTensorDescriptor(p.x);
    if (p.w) miopenDestroyTensorDescriptor(p.w);
    if (p.y) miopenDestroyTensorDescriptor(p.y);
    if (p.conv) miopenDestroyConvolutionDescriptor(p.conv);
  }
  g_problems.clear();
  if (g_ws) (void)hipFree(g_ws);
  g_ws = nullptr;
  g_ws_cap = 0;
  if (g_handle) miopenDestroy(g_handle);
  g_handle = nullptr;
}

}  // extern "C"
