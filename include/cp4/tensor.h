// tensor_shape and Tensor: the reference's container types
// (Cuda_kernels/Tensor.cuh:10-44) for the MI355X build.
//
// The reference allocates with cudaMallocManaged so that one pointer serves
// host code and kernels.  On MI355X managed memory without XNACK stays in host
// RAM, so kernels reading it would run at link speed; this Tensor keeps
// m_data in pinned host memory (host code dereferences it exactly as the
// reference's tests do, Cuda_kernels/test/test_Tensor.cpp.cu:17) and owns an
// explicit HBM mirror that the CP:: operators fill and read back.
#ifndef CP4_TENSOR_H
#define CP4_TENSOR_H

#include <cstddef>
#include <initializer_list>
#include <tuple>
#include <vector>

// Same nine fields, order and lexicographic ordering as Tensor.cuh:10-25.
struct tensor_shape {
  unsigned N = 0;
  unsigned H = 0;
  unsigned W = 0;
  unsigned pad = 0;
  unsigned T = 0;
  unsigned C = 0;
  unsigned Y = 0;
  unsigned X = 0;
  unsigned Rank = 0;

  friend bool operator<(const tensor_shape l, const tensor_shape r) {
    return std::tie(l.N, l.H, l.W, l.pad, l.T, l.C, l.Y, l.X, l.Rank) <
           std::tie(r.N, r.H, r.W, r.pad, r.T, r.C, r.Y, r.X, r.Rank);
  }
};

class Tensor {
 public:
  float* m_data;                 // pinned host memory, zero-initialised
  std::vector<unsigned> shape;

  Tensor(std::initializer_list<unsigned>);
  explicit Tensor(const std::vector<unsigned>& shape);
  Tensor(Tensor const&);            // deep copy (Tensor.cu:18-23)
  Tensor(Tensor&&) noexcept;
  Tensor& operator=(Tensor const&); // deep copy, also of the shape
  Tensor& operator=(Tensor&&) noexcept;
  ~Tensor();

  size_t size() const;              // product of the dims, as size_t
  size_t order() const { return shape.size(); }

  // HBM mirror.  device() allocates it on first use; upload()/download() copy
  // the whole tensor synchronously.  Kernels only ever see device().
  float* device() const;
  void upload() const;
  void download();

 private:
  mutable float* d_data_ = nullptr;
  void allocate(size_t n);
  void release();
};

#endif  // CP4_TENSOR_H
