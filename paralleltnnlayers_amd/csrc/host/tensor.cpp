// Tensor: pinned host buffer + explicit HBM mirror, through the C ABI only.
#include "cp4/tensor.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "cp4/capi.h"

namespace {
void check(cp4_status st, const char* what) {
  if (st == CP4_OK) return;
  // same policy as the reference's ErrChk (Cuda_kernels/cp4Conv2dForward.cu:10-19)
  std::fprintf(stderr, "cp4 Tensor: %s: %s (%s)\n", what, cp4_status_string(st),
               cp4_last_error_message());
  std::exit((int)st);
}
size_t count(const std::vector<unsigned>& shape) {
  size_t n = 1;
  for (unsigned d : shape) n *= d;
  return n;
}
}  // namespace

void Tensor::allocate(size_t n) {
  m_data = nullptr;
  d_data_ = nullptr;
  if (n == 0) return;
  void* p = nullptr;
  check(cp4_host_malloc(&p, n * sizeof(float)), "pinned allocation");
  m_data = static_cast<float*>(p);
}

void Tensor::release() {
  if (m_data) check(cp4_host_free(m_data), "host free");
  if (d_data_) check(cp4_device_free(d_data_), "device free");
  m_data = nullptr;
  d_data_ = nullptr;
}

Tensor::Tensor(std::initializer_list<unsigned> l) : shape(l) {
  allocate(size());
  if (m_data) std::memset(m_data, 0, size() * sizeof(float));  // Tensor.cu:14
}

Tensor::Tensor(const std::vector<unsigned>& s) : shape(s) {
  allocate(size());
  if (m_data) std::memset(m_data, 0, size() * sizeof(float));
}

Tensor::Tensor(Tensor const& other) : shape(other.shape) {
  allocate(size());
  if (m_data) std::memcpy(m_data, other.m_data, size() * sizeof(float));
}

Tensor::Tensor(Tensor&& other) noexcept
    : m_data(other.m_data), shape(std::move(other.shape)), d_data_(other.d_data_) {
  other.m_data = nullptr;
  other.d_data_ = nullptr;
  other.shape.clear();
}

Tensor& Tensor::operator=(Tensor const& other) {
  if (this == &other) return *this;
  if (size() != other.size() || !m_data) {
    release();
    shape = other.shape;
    allocate(size());
  } else {
    shape = other.shape;
  }
  if (m_data) std::memcpy(m_data, other.m_data, size() * sizeof(float));
  return *this;
}

Tensor& Tensor::operator=(Tensor&& other) noexcept {
  if (this == &other) return *this;
  release();
  m_data = other.m_data;
  d_data_ = other.d_data_;
  shape = std::move(other.shape);
  other.m_data = nullptr;
  other.d_data_ = nullptr;
  other.shape.clear();
  return *this;
}

Tensor::~Tensor() { release(); }

size_t Tensor::size() const { return shape.empty() ? 0 : count(shape); }

float* Tensor::device() const {
  if (!d_data_ && size()) {
    void* p = nullptr;
    check(cp4_device_malloc(&p, size() * sizeof(float)), "device allocation");
    d_data_ = static_cast<float*>(p);
  }
  return d_data_;
}

void Tensor::upload() const {
  if (!size()) return;
  check(cp4_memcpy_h2d(device(), m_data, size() * sizeof(float), nullptr), "upload");
  check(cp4_stream_synchronize(nullptr), "upload sync");
}

void Tensor::download() {
  if (!size()) return;
  check(cp4_memcpy_d2h(m_data, device(), size() * sizeof(float), nullptr), "download");
  // synchronises, and reports a kernel that gave up a wait between its waves: what
  // was copied is incomplete then
  check(cp4_device_status(nullptr, nullptr), "download");
}
